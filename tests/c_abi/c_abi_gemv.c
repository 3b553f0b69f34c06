/* The C ABI of include/crow_hip.h driven from plain C, with no Python and no torch in the process: what a cgo / Rust FFI
 * caller does.  init -> kernel lookup -> device buffers -> repack at load -> launch with library-chosen dims -> status ->
 * download, checked against the CPU oracle (test infrastructure, linked only by this test program).
 * Prints "c_abi ok ..." and exits 0 on success. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/crow_hip.h"
#include "../../oracle/nvfp4_oracle.h"

#define CK(call)                                                                      \
    do {                                                                              \
        int rc_ = (call);                                                             \
        if (rc_ != 0) {                                                               \
            fprintf(stderr, "%s -> %d (%s)\n", #call, rc_, crow_hip_error_string(rc_)); \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

static uint64_t sm_state = 0x1234;
static uint64_t splitmix(void) {
    uint64_t z = (sm_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

int main(void) {
    const uint32_t rows = 200, cols = 1280; /* not multiples of the 64 x 256 tile: padded by the repacker */
    const float gs = 7.0e-4f;
    const size_t nbytes = crow_hip_container_bytes(rows, cols);
    if (nbytes != orc_byte_len(rows, cols)) return 2;
    uint8_t* w = (uint8_t*)malloc(nbytes);
    float* x = (float*)malloc(cols * sizeof(float));
    float *y = (float*)malloc(rows * sizeof(float)), *ref = (float*)malloc(rows * sizeof(float));
    for (size_t b = 0; b < nbytes / 36; b++) {
        for (int i = 0; i < 4; i++) w[b * 36 + i] = (uint8_t)(0x28 + splitmix() % 24); /* valid scale bytes */
        for (int i = 4; i < 36; i++) w[b * 36 + i] = (uint8_t)splitmix();
    }
    for (uint32_t i = 0; i < cols; i++) x[i] = (float)((double)(splitmix() >> 11) / 9007199254740992.0 * 4.0 - 2.0);

    CK(crow_hip_init(0));
    char name[256];
    CK(crow_hip_device_name(name, sizeof name));
    crow_module_t mod;
    CK(crow_hip_module_load(&mod));
    crow_fn_t f, missing;
    CK(crow_hip_module_get(mod, "gemv_nvfp4_w", &f));
    if (crow_hip_module_get(mod, "no_such_kernel", &missing) != CROW_ERR_KERNEL_MISSING) return 3;
    if (crow_hip_function_arg_count(f) != 6) return 4;

    void *d_raw, *d_w, *d_x, *d_y, *d_gs, *d_k, *d_rows;
    CK(crow_hip_alloc(nbytes, &d_raw));
    CK(crow_hip_alloc(crow_hip_tiled_bytes(rows, cols), &d_w));
    CK(crow_hip_alloc(cols * sizeof(float), &d_x));
    CK(crow_hip_alloc(rows * sizeof(float), &d_y));
    CK(crow_hip_alloc(sizeof(float), &d_gs));
    CK(crow_hip_alloc(sizeof(int), &d_k));
    CK(crow_hip_alloc(sizeof(int), &d_rows));
    const int k_word = (int)cols, rows_word = (int)rows;
    CK(crow_hip_upload(d_raw, w, nbytes));
    CK(crow_hip_upload(d_x, x, cols * sizeof(float)));
    CK(crow_hip_upload(d_gs, &gs, sizeof gs));
    CK(crow_hip_upload(d_k, &k_word, sizeof k_word));
    CK(crow_hip_upload(d_rows, &rows_word, sizeof rows_word));
    CK(crow_hip_repack_nvfp4(d_raw, rows, cols, d_w)); /* the one load-time call the reference does not have */
    CK(crow_hip_free(d_raw));

    crow_dims d;
    CK(crow_hip_launch_dims("gemv_nvfp4_w", rows, cols, 1, &d));
    /* launch_v(k.f("gemv_nvfp4_w"), gx, gy, gz, bx, &[w, x, gs, y, k_p, rows_p]): every value a device address */
    const uint64_t vals[6] = {(uint64_t)(uintptr_t)d_w, (uint64_t)(uintptr_t)d_x,  (uint64_t)(uintptr_t)d_gs,
                              (uint64_t)(uintptr_t)d_y, (uint64_t)(uintptr_t)d_k, (uint64_t)(uintptr_t)d_rows};
    if (crow_hip_launch(f, d.gx, d.gy, d.gz, d.bx, vals, 5, NULL) != CROW_ERR_ARG_COUNT) return 5; /* wrong count is refused */
    CK(crow_hip_launch(f, d.gx, d.gy, d.gz, d.bx, vals, 6, NULL));
    CK(crow_hip_status()); /* synchronises; a refused shape or a short workspace would show here */
    CK(crow_hip_download(y, d_y, rows * sizeof(float)));

    if (orc_gemv(w, rows, cols, gs, x, 1, ref, 1, 0) != 0) return 6;
    double rms = 0.0, worst = 0.0;
    for (uint32_t r = 0; r < rows; r++) rms += (double)ref[r] * ref[r];
    rms = sqrt(rms / rows);
    for (uint32_t r = 0; r < rows; r++) {
        const double den = fmax(fabs(ref[r]), 1e-2 * rms), e = fabs((double)y[r] - ref[r]) / den;
        if (e > worst) worst = e;
    }
    CK(crow_hip_free(d_w)); CK(crow_hip_free(d_x)); CK(crow_hip_free(d_y)); CK(crow_hip_free(d_gs)); CK(crow_hip_free(d_k)); CK(crow_hip_free(d_rows));
    CK(crow_hip_module_unload(mod));
    CK(crow_hip_shutdown());
    if (!(worst <= 1e-3)) {
        fprintf(stderr, "max relative error %.3g > 1e-3\n", worst);
        return 7;
    }
    printf("c_abi ok: %s, grid (%u,%u,%u) x %u, max relative error %.3g\n", name, d.gx, d.gy, d.gz, d.bx, worst);
    return 0;
}
