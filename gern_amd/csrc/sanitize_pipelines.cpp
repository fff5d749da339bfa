// Host-only exercise of the pipeline C ABI for sanitizer builds
// (`python gern_amd/build.py --sanitize`): every pipeline is composed, lowered,
// generated and compiled for gfx950 without a device, created and destroyed
// several times, and the error paths are taken.  No kernel runs.
#include "gern_pipelines.h"

#include <cstdio>
#include <cstring>
#include <initializer_list>

static int failures = 0;

static void expect(bool ok, const char *what) {
    if (!ok) {
        char buf[2048];
        gern_pipelines_last_error(buf, sizeof buf);
        std::printf("FAIL %s: %s\n", what, buf);
        failures++;
    }
}

int main() {
    const int compile_only = GERN_PIPELINE_COMPILE_ONLY;
    for (int round = 0; round < 3; round++) {
        gern_pipeline p = nullptr;
        for (int variant = 0; variant < 2; variant++) {
            for (int flags : {0, (int)GERN_PIPELINE_GEMM_OVERWRITE, (int)GERN_PIPELINE_GEMM_GENERAL_ONLY}) {
                expect(gern_gemm_create(variant, compile_only | flags, &p) == 0, "gemm create");
                expect(std::strlen(gern_pipeline_source(p)) > 0 && std::strlen(gern_pipeline_kernel_name(p)) > 0, "gemm source");
                float c = 0.f;
                expect(gern_gemm_run(p, &c, &c, &c, 1, 1, 1, nullptr) != 0, "compile-only pipeline must refuse to run");
                gern_pipeline_destroy(p);
            }
        }
        for (long ncol : {7L, 1000L, 1024L, 3072L, 4096L, 8192L}) {
            expect(gern_softmax_create(ncol, 1, compile_only, &p) == 0, "softmax create");
            gern_pipeline_destroy(p);
        }
        for (const char *pattern : {"x", "y", "xy", "xyx", "yxy"}) {
            expect(gern_blur_chain_create(pattern, 3, 6, 252, 1, compile_only, &p) == 0, "blur create");
            gern_pipeline_destroy(p);
        }
        expect(gern_blur_chain_create("xyx", 3, 8, 252, 4, compile_only | GERN_PIPELINE_NO_XCD_REMAP, &p) == 0, "blur, four wavefronts");
        gern_pipeline_destroy(p);
        for (long d : {32L, 96L, 128L, 256L}) {
            expect(gern_qk_softmax_create(d, d == 256 ? 1024 : 4096, compile_only, &p) == 0, "qk create");
            gern_pipeline_destroy(p);
        }
        expect(gern_blur_chain_create("xyx", 3, 4, 224, 1, compile_only, &p) == 0, "blur, line-aligned store windows");
        gern_pipeline_destroy(p);
        expect(gern_qk_softmax_create(128, 4096, compile_only | GERN_PIPELINE_QK_ROW_BLOCKS, &p) == 0, "qk row blocks");
        gern_pipeline_destroy(p);
        for (int schedule : {3, 6, 10}) {
            expect(gern_gemm_schedule_create(schedule, compile_only, &p) == 0, "gemm schedule create");
            gern_pipeline_destroy(p);
        }
        expect(gern_gemm_schedule_create(4, compile_only, &p) != 0 && p == nullptr, "bad schedule");
        // argument errors leave no pipeline behind
        expect(gern_gemm_create(7, compile_only, &p) != 0 && p == nullptr, "bad variant");
        expect(gern_softmax_create(0, 1, compile_only, &p) != 0 && p == nullptr, "bad width");
        expect(gern_blur_chain_create("xz", 3, 6, 252, 1, compile_only, &p) != 0 && p == nullptr, "bad pattern");
        expect(gern_qk_softmax_create(100, 4096, compile_only, &p) != 0 && p == nullptr, "bad head dimension");
        expect(gern_blur_chain_create(nullptr, 3, 6, 252, 1, compile_only, &p) != 0, "null pattern");
    }
    std::printf(failures ? "sanitize_pipelines: %d failures\n" : "sanitize_pipelines: ok\n", failures);
    return failures != 0;
}
