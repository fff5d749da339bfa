/* A host written in plain C that uses nothing but the C ABI
 * (include/gern_pipelines.h, include/gern_hip.h): create the three-stage blur
 * chain, run it on an image, copy the result back and compare it with the
 * same arithmetic done on the host.
 *
 *   gcc -std=c99 -Iinclude examples/blur_c_host.c -Lgern_amd -lgern_pipelines -lgern -lgern_hip \
 *       -Wl,-rpath,$PWD/gern_amd -o blur_c_host && ./blur_c_host
 *
 * With --compile-only it builds the pipeline for gfx950 without a device and
 * prints the name of the generated kernel (what a machine without a GPU can
 * check).  Exit status 0 = as expected. */
#include "gern_hip.h"
#include "gern_pipelines.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int fail(const char *what) {
    char msg[4096];
    gern_pipelines_last_error(msg, sizeof msg);
    fprintf(stderr, "%s: %s\n", what, msg);
    gern_hip_last_error(msg, sizeof msg);
    if (msg[0] != '\0') {
        fprintf(stderr, "  runtime: %s\n", msg);
    }
    return 1;
}

/* o[i][j] = (0 + a + b + c) / 3 along a row (dx = 1) or down a column (dx = 0),
 * the arithmetic of apps/blur/blur.cpp:11-25 of the reference. */
static void blur_host(const float *in, int rows, int cols, int along_x, float *out) {
    const int orows = along_x ? rows : rows - 2, ocols = along_x ? cols - 2 : cols;
    for (int i = 0; i < orows; i++) {
        for (int j = 0; j < ocols; j++) {
            const float *p = in + (size_t)i * cols + j;
            const int step = along_x ? 1 : cols;
            out[(size_t)i * ocols + j] = (0.0f + p[0] + p[step] + p[2 * step]) / 3;
        }
    }
}

int main(int argc, char **argv) {
    const int compile_only = argc > 1 && strcmp(argv[1], "--compile-only") == 0;
    const int rows = 300, cols = 700;
    gern_pipeline blur = NULL;
    if (gern_blur_chain_create("xyx", 3, 6, 252, 1, compile_only ? GERN_PIPELINE_COMPILE_ONLY : 0, &blur) != 0) {
        return fail("gern_blur_chain_create");
    }
    printf("kernel: %s\n", gern_pipeline_kernel_name(blur));
    if (compile_only) {
        float dummy = 0.0f;
        /* a pipeline that was only compiled must refuse to run */
        const int refused = gern_blur_chain_run(blur, &dummy, rows, cols, cols, &dummy, cols - 4, NULL) != 0;
        gern_pipeline_destroy(blur);
        return refused ? 0 : 1;
    }

    const int orows = rows - 2, ocols = cols - 4;
    float *img = malloc(sizeof(float) * rows * cols);
    float *got = malloc(sizeof(float) * orows * ocols);
    float *t1 = malloc(sizeof(float) * rows * (cols - 2));
    float *t2 = malloc(sizeof(float) * orows * (cols - 2));
    float *want = malloc(sizeof(float) * orows * ocols);
    unsigned state = 12345u;
    for (int i = 0; i < rows * cols; i++) {
        state = state * 1664525u + 1013904223u;
        img[i] = (float)(state >> 8) * (1.0f / 16777216.0f);
    }
    blur_host(img, rows, cols, 1, t1);
    blur_host(t1, rows, cols - 2, 0, t2);
    blur_host(t2, orows, cols - 2, 1, want);

    void *d_img = NULL, *d_out = NULL;
    if (gern_hip_malloc(&d_img, sizeof(float) * rows * cols) != 0 || gern_hip_malloc(&d_out, sizeof(float) * orows * ocols) != 0 ||
        gern_hip_memcpy_h2d(d_img, img, sizeof(float) * rows * cols) != 0) {
        return fail("device buffers");
    }
    if (gern_blur_chain_run(blur, d_img, rows, cols, cols, d_out, ocols, NULL) != 0) {
        return fail("gern_blur_chain_run");
    }
    if (gern_hip_sync() != 0 || gern_hip_memcpy_d2h(got, d_out, sizeof(float) * orows * ocols) != 0) {
        return fail("copy back");
    }
    long mismatches = 0;
    for (long i = 0; i < (long)orows * ocols; i++) {
        mismatches += memcmp(&got[i], &want[i], sizeof(float)) != 0;
    }
    printf("%d x %d outputs, %ld differ from the host arithmetic\n", orows, ocols, mismatches);
    gern_hip_free(d_img);
    gern_hip_free(d_out);
    gern_pipeline_destroy(blur);
    free(img); free(got); free(t1); free(t2); free(want);
    return mismatches == 0 ? 0 : 1;
}
