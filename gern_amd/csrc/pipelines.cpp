// C ABI over the fused pipelines (include/gern_pipelines.h).  Everything here
// is written against Gern's C++ API, the way a user application is: declare
// data structures, compose annotated functions, compile with a Runner,
// evaluate with the caller's buffers.
#include "gern_pipelines.h"

#include "annot/blur.h"
#include "annot/lds_matrix.h"
#include "annot/mm.h"
#include "annot/qk_softmax.h"
#include "annot/softmax.h"
#include "gern/codegen/codegen.h"
#include "gern_hip.h"

#include <dlfcn.h>

#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <cstdlib>
#include <memory>
#include <sstream>
#include <string>

using namespace gern;

namespace {

thread_local std::string g_error;

int fail(const std::string &msg) {
    g_error = msg;
    return 1;
}

// Directory that holds this library; the gernel headers live next to it.
// Where gernels/ and annot/ are: the directory of this library, unless
// GERN_PACKAGE_DIR names another one (a library built or installed elsewhere).
std::string packageDir() {
    if (const char *dir = std::getenv("GERN_PACKAGE_DIR")) {
        if (*dir != '\0') {
            return dir;
        }
    }
    Dl_info info;
    if (dladdr((const void *)&packageDir, &info) && info.dli_fname) {
        std::string path(info.dli_fname);
        auto slash = path.rfind('/');
        return slash == std::string::npos ? "." : path.substr(0, slash);
    }
    return ".";
}

// GERN_EXPERIMENTS=1 lets the environment change what the pipelines are built from (extra compiler
// options, other band heights and wavefront counts): for measurements, never needed for results.
bool experiments() {
    const char *v = std::getenv("GERN_EXPERIMENTS");
    return v != nullptr && std::string(v) == "1";
}

AbstractDataTypePtr f32(const std::string &name, annot::MatrixF32::Role role) {
    return AbstractDataTypePtr(new const annot::MatrixF32(name, role));
}

}  // namespace

struct gern_pipeline_s {
    enum Kind { BLUR, SOFTMAX, GEMM_F32, GEMM_BF16, QK_SOFTMAX, GEMM_SCHEDULE } kind;
    std::unique_ptr<Runner> runner;  // null in compile-only mode
    std::unique_ptr<Runner> exact;   // GEMM: the direct-to-LDS matrix-core kernel (rows of A in whole 16-byte pieces)
    std::unique_ptr<Runner> tail;    // fp32 GEMM in overwrite mode: C += of the last K % 4 columns
    bool accumulate = true;          // GEMM: C += A * B (false: C = A * B)
    int create_flags = 0;
    std::string source;
    std::string kernel_name;
    std::string exact_source, exact_kernel_name;
    bool last_run_exact = false;
    // blur
    int64_t nx = 0, ny = 0, stride = 0;
    // softmax / qk
    int64_t ncol = 0;
    int64_t head_dim = 0;
    // qk on 256 x 256 tiles: the memory through which the workgroups of a row block exchange row statistics
    bool qk_tiles = false;
    void *qk_scratch = nullptr;
    // the exchange memory of the library (csrc/qk_no_alloc.hip) on this pipeline's GPU; null if it has none
    void *qk_shared_scratch = nullptr;
    bool qk_used_shared = false;      // a run went through qk_shared_scratch since the last gern_pipeline_faults
    bool qk_default_period = true;    // built with the tag period every user of the shared memory agrees on
    void *last_stream = nullptr;
    // parameter names
    std::vector<std::string> names;
};

namespace {

// The rule of gernels/qk_softmax.h (qk_waves): wavefronts per row block.
int64_t qkWaves(int64_t n) {
    return (n >= 2048 && n % 512 == 0) ? 8 : 4;
}

// Generates (and, unless compile-only, loads) the program.
int finish(gern_pipeline_s *p, Composable program, int flags, int min_waves_per_simd = 0, int xcd_band_rows = 0) {
    std::string include = "-I " + packageDir();
    if (const char *extra = std::getenv("GERN_PIPELINE_EXTRA_OPTIONS"); extra != nullptr && experiments()) {
        include += std::string(" ") + extra;  // e.g. "-DNAME=value"
        p->qk_default_period = std::string(extra).find("GERN_QK_TAG_PERIOD") == std::string::npos;
    }
    try {
        if (flags & GERN_PIPELINE_COMPILE_ONLY) {
            codegen::GeneratorOptions go;
            go.xcd_remap = !(flags & GERN_PIPELINE_NO_XCD_REMAP);
            go.xcd_tile_blocks = (flags & GERN_PIPELINE_XCD_TILE_BLOCKS) != 0;
            go.xcd_band_rows = xcd_band_rows;
            go.min_waves_per_simd = min_waves_per_simd;
            codegen::CodeGenerator cg(std::nullopt, go);
            p->source = cg.generate_code(program);
            p->kernel_name = cg.getLaunchPlan().name_expression;
            p->names = cg.getArgumentOrder();
            // the same options the Runner would pass: "-I <dir>" and whatever GERN_PIPELINE_EXTRA_OPTIONS adds
            std::vector<std::string> words;
            std::istringstream in(include);
            for (std::string w; in >> w;) {
                if (w == "-I" && (in >> w)) {
                    w = "-I" + w;
                }
                words.push_back(w);
            }
            std::vector<const char *> opts;
            for (const auto &w : words) {
                opts.push_back(w.c_str());
            }
            const char *names[1] = {p->kernel_name.c_str()};
            size_t size = 0;
            if (gern_hip_compile_only(p->source.c_str(), names, 1, opts.data(), (int)opts.size(), "gfx950", &size) != 0) {
                std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
                gern_hip_last_error(msg.data(), msg.size());
                return fail("Compilation Failed\n" + msg);
            }
            return 0;
        }
        p->runner = std::make_unique<Runner>(program);
        Runner::Options options;
        options.filename = "";  // keep the source in memory only
        options.include = include;
        options.xcd_remap = !(flags & GERN_PIPELINE_NO_XCD_REMAP);
        options.xcd_tile_blocks = (flags & GERN_PIPELINE_XCD_TILE_BLOCKS) != 0;
        options.xcd_band_rows = xcd_band_rows;
        options.min_waves_per_simd = min_waves_per_simd;
        p->runner->compile(options);
        p->source = p->runner->getSource();
        p->names = p->runner->getArgumentOrder();
        return 0;
    } catch (const std::exception &e) {
        return fail(e.what());
    }
}

}  // namespace

// csrc/qk_no_alloc.hip: the address of the library's exchange memory on the current GPU (looked up, once per
// GPU, on the first call).  Weak: a build of this file without that object has no such memory.
extern "C" __attribute__((weak, visibility("hidden"))) int gern_detail_qk_shared_scratch(void **out);

extern "C" {

int gern_blur_chain_create(const char *pattern, int64_t stride, int64_t tile_rows, int64_t tile_cols,
                           int waves_per_block, int flags, gern_pipeline *out) {
    if (out == nullptr || pattern == nullptr) {
        return fail("gern_blur_chain_create: null argument");
    }
    *out = nullptr;
    const std::string pat(pattern);
    int64_t nx = 0, ny = 0;
    for (char ch : pat) {
        if (ch == 'x') {
            nx++;
        } else if (ch == 'y') {
            ny++;
        } else {
            return fail("gern_blur_chain_create: pattern must consist of 'x' and 'y'");
        }
    }
    if (pat.empty() || stride < 1 || stride > 5 || tile_rows < 1 || tile_cols < 1 || waves_per_block < 1 ||
        waves_per_block > 16) {
        return fail("gern_blur_chain_create: bad stride, tile or workgroup shape");
    }
    if (tile_cols % 4 != 0 || tile_cols + nx * (stride - 1) > 256) {
        return fail("gern_blur_chain_create: tile_cols must be a multiple of 4 and tile_cols + halo <= 256");
    }
    auto p = std::make_unique<gern_pipeline_s>();
    p->kind = gern_pipeline_s::BLUR;
    p->nx = nx;
    p->ny = ny;
    p->stride = stride;
    try {
        // Tiles a whole number of 128-byte lines wide that leave 28 columns
        // of the wavefront's 256 free write line-aligned windows of the result
        // (gernels/wave_tile.h, store_wave_lines).
        const bool lines = tile_cols % 32 == 0 && tile_cols + 28 + nx * (stride - 1) <= 256 &&
                           !(flags & GERN_PIPELINE_BLUR_PLAIN_STORES);
        auto input = f32("input", lines ? annot::MatrixF32::INPUT_WIDE : annot::MatrixF32::INPUT);
        auto output = f32("output", lines ? annot::MatrixF32::OUTPUT_LINES : annot::MatrixF32::OUTPUT);
        Variable stride_v("stride"), row("row"), col("col"), col_block("col_block"), wave("wave");
        std::vector<Composable> stages;
        AbstractDataTypePtr prev = input;
        for (size_t s = 0; s < pat.size(); s++) {
            AbstractDataTypePtr next =
                (s + 1 == pat.size()) ? output : f32("stage" + std::to_string(s), annot::MatrixF32::TEMP);
            std::map<std::string, Variable> bind{{"stride", stride_v.bind(stride)}};
            if (pat[s] == 'x') {
                annot::BlurX f{prev, next};
                stages.push_back(f[bind](prev, next));
            } else {
                annot::BlurY f{prev, next};
                stages.push_back(f[bind](prev, next));
            }
            prev = next;
        }
        Composable chain(new const Computation(stages));
        Composable program;
        if (waves_per_block == 1) {
            program = Global((Tile(output["row"], row.bind(tile_rows)) || Grid::BLOCK_Y)(
                                 (Tile(output["col"], col.bind(tile_cols)) || Grid::BLOCK_X)(chain)),
                             {{Grid::BLOCK_DIM_X, wave.bind(Grid::kWavefrontSize)}});
        } else {
            program = Global((Tile(output["row"], row.bind(tile_rows)) || Grid::BLOCK_Y)(
                (Tile(output["col"], col_block.bind(tile_cols * waves_per_block)) || Grid::BLOCK_X)(
                    (Tile(output["col"], col.bind(tile_cols)) || Grid::WARP_X)(chain))));
        }
        // XCD order: bands of about 64 output rows (16 rows of 4-row tiles) dealt to the XCDs in turn.  Halo rows
        // are shared inside a band through that XCD's L2 (one in sixteen tile rows has its lower neighbour on
        // another XCD), and the eight XCDs stream through one 16 MiB window of an 8192-wide image together
        // instead of through eight places 32 MiB apart: 8192^2 x,y,x over rotating buffers 92.6 -> 90.3 us,
        // same buffers 86 -> 78-86 us (measured in one process; bands of 8 rows of tiles 89.8 us, of 32 and
        // more 94-105 us, one tile row per band 108 us).  With GERN_EXPERIMENTS=1, GERN_BLUR_BAND_ROWS
        // overrides it (0 = one contiguous run of tiles per XCD).
        int band_rows = (int)std::max<int64_t>(1, 64 / tile_rows);
        if (const char *v = std::getenv("GERN_BLUR_BAND_ROWS"); v != nullptr && experiments()) {
            band_rows = std::max(0, std::atoi(v));
        }
        int rc = finish(p.get(), program, flags, 0, band_rows);
        if (rc != 0) {
            return rc;
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    *out = p.release();
    return 0;
}

int gern_blur_chain_run(gern_pipeline p, const float *in, int64_t rows, int64_t cols, int64_t ld_in,
                        float *out, int64_t ld_out, void *stream) {
    if (p == nullptr || p->kind != gern_pipeline_s::BLUR || in == nullptr || out == nullptr) {
        return fail("gern_blur_chain_run: bad pipeline or null buffer");
    }
    if (!p->runner) {
        return fail("gern_blur_chain_run: the pipeline was created compile-only");
    }
    const int64_t out_rows = rows - p->ny * (p->stride - 1);
    const int64_t out_cols = cols - p->nx * (p->stride - 1);
    if (out_rows <= 0 || out_cols <= 0 || ld_in < cols || ld_out < out_cols) {
        return fail("gern_blur_chain_run: the image is smaller than the stencil footprint, or a bad row stride");
    }
    hip::MatrixF32 input{const_cast<float *>(in), rows, cols, ld_in};
    hip::MatrixF32 output{out, out_rows, out_cols, ld_out};
    try {
        p->runner->setStream(stream);
        p->runner->evaluate({{"input", &input}, {"output", &output}});
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    return 0;
}

int gern_softmax_create(int64_t ncol, int64_t rows_per_wave, int flags, gern_pipeline *out) {
    if (out == nullptr) {
        return fail("gern_softmax_create: null argument");
    }
    *out = nullptr;
    if (ncol < 1 || ncol > GERN_SOFTMAX_MAX_COLS || rows_per_wave < 1) {
        return fail("gern_softmax_create: ncol must be in [1, GERN_SOFTMAX_MAX_COLS = 65536] and rows_per_wave positive");
    }
    // A row is cut into equal pieces of whole 256-column chunks, at least 512
    // columns each, one per wavefront of the workgroup that owns the row (8, 4
    // or 2 of them): many short wavefronts overlap the loads of one row with
    // the stores of another (8192 x 4096: 46 -> 39.5 us, 4096 x 8192: 68 -> 41.5;
    // sixteen wavefronts of 256 columns: 54 us).  Widths that do not divide
    // that way keep one wavefront per row.
    // A row wider than 8192 columns does not fit the registers of one wavefront (32 chunks of 256 columns,
    // 128 values per lane): it is cut into 4, 8 or 16 pieces of at most 4096 columns, whatever its width (the
    // last pieces of a width that does not divide are partly or wholly unused, gernels/softmax.h BlockTile).
    int64_t waves = 1;
    for (int64_t w : {8, 4, 2}) {
        if (ncol % (w * 256) == 0 && ncol / w >= 512) {
            waves = w;
            break;
        }
    }
    if (ncol > 8192) {
        waves = ncol <= 16384 ? 4 : ncol <= 32768 ? 8 : 16;
    }
    if (const char *forced = std::getenv("GERN_SOFTMAX_WAVES"); forced != nullptr && experiments()) {
        waves = std::atoll(forced);
        if ((waves != 1 && waves != 2 && waves != 4 && waves != 8 && waves != 16) || ncol % (4 * waves) != 0) {
            return fail("GERN_SOFTMAX_WAVES must be 1, 2, 4, 8 or 16 and divide the row into 16-byte pieces");
        }
    }
    if (rows_per_wave * (((ncol + waves - 1) / waves + 255) / 256) > 32) {
        return fail("gern_softmax_create: a wavefront holds at most 32 x 256 columns of rows in registers");
    }
    auto p = std::make_unique<gern_pipeline_s>();
    p->kind = gern_pipeline_s::SOFTMAX;
    p->ncol = ncol;
    try {
        using M = annot::MatrixF32;
        auto matrix = [&](const char *name, M::Role role) {
            return waves == 1 ? f32(name, role)
                              : AbstractDataTypePtr(new const annot::BlockRowsF32(name, role, (int)waves));
        };
        auto input = matrix("input", M::INPUT);
        auto output = matrix("output", M::OUTPUT);
        auto shifted = matrix("shifted", M::TEMP);
        auto expd = matrix("expd", M::TEMP);
        auto row_max = AbstractDataTypePtr(new const annot::WaveVec("row_max"));
        auto row_sum = AbstractDataTypePtr(new const annot::WaveVec("row_sum"));
        Variable rows("rows"), ncol_v("ncol"), threads("threads");
        annot::MaxRow max_row{input, row_max};
        annot::SubtractVec sub{row_max, input, shifted};
        annot::ExpMatrix ex{shifted, expd};
        annot::SumRow sum_row{expd, row_sum};
        annot::DivideVec div{row_sum, expd, output};
        std::map<std::string, Variable> width{{"ncol", ncol_v.bind(ncol)}};
        Composable program =
            Global((Tile(output["row"], rows.bind(rows_per_wave)) || Grid::BLOCK_X)(
                       Tile(output["col"], ncol_v.bind(ncol))(max_row[width](row_max, input), sub(row_max, input, shifted),
                                                              ex(shifted, expd), sum_row[width](row_sum, expd),
                                                              div(row_sum, expd, output))),
                   {{Grid::BLOCK_DIM_X, threads.bind(Grid::kWavefrontSize * waves)}});
        // Rows are contiguous and independent: plain launch order already
        // streams through memory, and measures faster than the XCD order
        // (8192 x 4096 over rotating buffers: 45.3 us; bands of 4, 16, 64, 256
        // rows dealt to the XCDs in turn 46.3, 45.7, 46.9, 47.9 us).
        int rc = finish(p.get(), program, flags | GERN_PIPELINE_NO_XCD_REMAP);
        if (rc != 0) {
            return rc;
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    *out = p.release();
    return 0;
}

int gern_softmax_run(gern_pipeline p, const float *in, float *out, int64_t rows, int64_t ld, void *stream) {
    if (p == nullptr || p->kind != gern_pipeline_s::SOFTMAX || in == nullptr || out == nullptr) {
        return fail("gern_softmax_run: bad pipeline or null buffer");
    }
    if (!p->runner) {
        return fail("gern_softmax_run: the pipeline was created compile-only");
    }
    if (rows < 1 || ld < p->ncol) {
        return fail("gern_softmax_run: bad shape");
    }
    hip::MatrixF32 input{const_cast<float *>(in), rows, p->ncol, ld};
    hip::MatrixF32 output{out, rows, p->ncol, ld};
    try {
        p->runner->setStream(stream);
        p->runner->evaluate({{"input", &input}, {"output", &output}});
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    return 0;
}

namespace {

// Tile(i)(Tile(j)(Reduce(k)(matrix_multiply))) for one choice of data
// structures; one call of the gernel walks a whole 4096-deep K chunk.
Composable gemmProgram(annot::MatrixOperand::Element element, bool exact, annot::MatrixAccumulator::Engine engine,
                       bool accumulate, int64_t bm, int64_t bn, int64_t threads_per_block, int64_t lds) {
    auto A = AbstractDataTypePtr(new const annot::MatrixOperand("A", element, exact));
    auto B = AbstractDataTypePtr(new const annot::MatrixOperand("B", element, exact));
    auto C = AbstractDataTypePtr(new const annot::MatrixAccumulator("C", engine, accumulate));
    Variable ti("ti"), tj("tj"), tk("tk"), k_dim("k_dim"), threads("threads"), smem("smem");
    annot::MatrixMultiply mm{A, B, C};
    Composable tiled = (Tile(C["row"], ti.bind(bm)) || Grid::BLOCK_Y)((Tile(C["col"], tj.bind(bn)) || Grid::BLOCK_X)(
        Reduce(k_dim, tk.bind(4096))(mm[{{"k_dim", k_dim}}](A, B, C))));
    if (lds == 0) {
        // A gernel that keeps its stages in static LDS asks for no dynamic LDS.
        return Global(tiled, {{Grid::BLOCK_DIM_X, threads.bind(threads_per_block)}});
    }
    return Global(tiled, {{Grid::BLOCK_DIM_X, threads.bind(threads_per_block)}}, smem.bind(lds));
}

}  // namespace

int gern_gemm_create(int variant, int flags, gern_pipeline *out) {
    if (out == nullptr) {
        return fail("gern_gemm_create: null argument");
    }
    *out = nullptr;
    if (variant != 0 && variant != 1) {
        return fail("gern_gemm_create: variant must be 0 (fp32) or 1 (bf16 in, fp32 accumulate)");
    }
    auto p = std::make_unique<gern_pipeline_s>();
    p->kind = variant == 1 ? gern_pipeline_s::GEMM_BF16 : gern_pipeline_s::GEMM_F32;
    const bool accumulate = !(flags & GERN_PIPELINE_GEMM_OVERWRITE);
    p->accumulate = accumulate;
    p->create_flags = flags;
    try {
        const bool bf16 = variant == 1;
        const auto element = bf16 ? annot::MatrixOperand::BF16 : annot::MatrixOperand::F32;
        // Plain workgroup order: the hardware deals consecutive ids to the 8 XCDs in
        // turn, so the tiles that run on one XCD at a time form a block several tile
        // rows high and several tile columns wide, which share A and B panels in that
        // XCD's L2.  Giving each XCD a contiguous band of ids (the renumbering that
        // helps the blur) makes that block one tile row of many columns: at 8192^3,
        // 33 panels per 32 tiles instead of 12, and 6 % slower (measured).
        // The kernels therefore take the order that makes the block explicit: 4 x 8 tiles per XCD at a
        // time, 12 panels per 32 tiles (at 4096^3 the plain order gives 2 x 16 tiles of 256 x 256, 18 panels).
        if (!(flags & GERN_PIPELINE_NO_XCD_REMAP)) {
            flags |= GERN_PIPELINE_XCD_TILE_BLOCKS;
        }
        flags |= GERN_PIPELINE_NO_XCD_REMAP;
        // The kernel for every shape.  bf16: four wavefronts, 256x256 tile, LDS of
        // gernels/mm.h mfma_lds_bytes(); fp32: vector-ALU FMAs, 128x128 tile, LDS
        // of fma_lds_bytes().
        int rc = bf16 ? finish(p.get(),
                               gemmProgram(element, false, annot::MatrixAccumulator::MFMA4, accumulate, 256, 256, 256,
                                           2 * (256 + 256) * 144),
                               flags)
                      : finish(p.get(),
                               gemmProgram(element, false, annot::MatrixAccumulator::FMA, accumulate, 128, 128, 256,
                                           2 * 2 * 16 * 132 * 4),
                               flags);
        if (rc == 0 && !(flags & GERN_PIPELINE_GEMM_GENERAL_ONLY)) {
            // The same program on data structures that promise rows of A in whole 16-byte pieces:
            // eight wavefronts, 256x256 tile on the matrix cores (also for fp32),
            // loads straight into LDS.  Those gernels keep their two stages in
            // static LDS (gernels/mm.h, mfma_direct / mfma_direct_f32): no dynamic LDS.
            gern_pipeline_s fast;
            // bf16: the 16 x 16 x 32 matrix instruction (it draws less power than 32 x 32 x 16 for the same
            // work, and the clock of this kernel is set by power); the other one stays selectable for
            // comparison.
            const bool wide_instruction = std::getenv("GERN_GEMM_BF16_32X32X16") != nullptr && experiments();
            rc = finish(&fast,
                        gemmProgram(element, true,
                                    !bf16            ? annot::MatrixAccumulator::MFMA8_F32 :
                                    wide_instruction ? annot::MatrixAccumulator::MFMA8 :
                                                       annot::MatrixAccumulator::MFMA16,
                                    accumulate, 256, 256, 512, 0),
                        flags);
            p->exact = std::move(fast.runner);
            p->exact_source = fast.source;
            p->exact_kernel_name = fast.kernel_name.empty() && p->exact ? p->exact->getKernelName() : fast.kernel_name;
            // The shape the pipeline is built for is the exact one.
            p->last_run_exact = true;
            if (rc == 0 && !bf16 && !accumulate) {
                // An fp32 product whose K is not a multiple of 4 is split in two launches (gern_gemm_run);
                // the second one ADDS the last columns even when the pipeline overwrites C.  Built here so
                // that a run never compiles.
                gern_pipeline_s rest;
                rc = finish(&rest, gemmProgram(element, false, annot::MatrixAccumulator::FMA, true, 128, 128, 256, 2 * 2 * 16 * 132 * 4),
                            flags);
                p->tail = std::move(rest.runner);
            }
        }
        if (rc != 0) {
            return rc;
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    *out = p.release();
    return 0;
}

int gern_gemm_run(gern_pipeline p, const void *A, const void *B, float *C, int64_t M, int64_t N, int64_t K,
                  void *stream) {
    if (p == nullptr || (p->kind != gern_pipeline_s::GEMM_F32 && p->kind != gern_pipeline_s::GEMM_BF16) ||
        A == nullptr || B == nullptr || C == nullptr) {
        return fail("gern_gemm_run: bad pipeline or null buffer");
    }
    if (!p->runner) {
        return fail("gern_gemm_run: the pipeline was created compile-only");
    }
    if (M < 1 || N < 1 || K < 1) {
        return fail("gern_gemm_run: bad shape");
    }
    if (p->kind == gern_pipeline_s::GEMM_BF16 && ((K % 8) != 0 || (N % 2) != 0)) {
        return fail("gern_gemm_run: the bf16 path needs K % 8 == 0 and N % 2 == 0 (16-byte rows of A, dword pairs of B)");
    }
    const uintptr_t pa = reinterpret_cast<uintptr_t>(A), pb = reinterpret_cast<uintptr_t>(B);
    if (p->kind == gern_pipeline_s::GEMM_BF16 ? ((pa & 15u) != 0 || (pb & 3u) != 0) : (((pa | pb) & 3u) != 0)) {
        return fail(p->kind == gern_pipeline_s::GEMM_BF16
                        ? "gern_gemm_run: the bf16 path reads A in 16-byte pieces and B in dwords: A must be 16-byte aligned, B 4-byte aligned"
                        : "gern_gemm_run: A and B must be 4-byte aligned");
    }
    if ((reinterpret_cast<uintptr_t>(C) & 3u) != 0) {
        return fail("gern_gemm_run: C must be 4-byte aligned");
    }
    // MatrixF32 and MatrixBF16 share their layout.
    hip::MatrixF32 a{static_cast<float *>(const_cast<void *>(A)), M, K, K};
    hip::MatrixF32 b{static_cast<float *>(const_cast<void *>(B)), K, N, N};
    hip::MatrixF32 c{C, M, N, N};
    int64_t k_dim = K;
    Runner *runner = p->runner.get();
    // The matrix-core gernels (gernels/mm.h, mfma_direct / mfma_direct_f32) read rows of A in whole 16-byte
    // pieces (bf16: K % 8 == 0, required above) with a 16-byte aligned A, and need row pitches (K for A, N for
    // B) within their 32-bit byte offsets; partial tiles and a partial last K stage are theirs too.  An fp32
    // product whose K is not a multiple of 4 is split: the first K - K % 4 columns of A (rows of B) go to the
    // matrix cores, the last one to three are added by the vector-ALU kernel in a second launch.
    const bool fp32 = p->kind == gern_pipeline_s::GEMM_F32;
    const int64_t k_main = fp32 ? K - K % 4 : K;
    const int64_t max_pitch = int64_t(1) << 20;  // gernels/mm.h, kMfmaMaxLd
    p->last_run_exact = p->exact && (pa & 15u) == 0 && k_main > 0 && K <= max_pitch && N <= max_pitch;
    try {
        if (!p->last_run_exact) {
            runner->setStream(stream);
            runner->evaluate({{"A", &a}, {"B", &b}, {"C", &c}, {"k_dim", &k_dim}});
            return 0;
        }
        a.col = k_main;
        b.row = k_main;
        k_dim = k_main;
        p->exact->setStream(stream);
        p->exact->evaluate({{"A", &a}, {"B", &b}, {"C", &c}, {"k_dim", &k_dim}});
        if (k_main < K) {
            Runner *rest = p->runner.get();  // accumulates unless the pipeline overwrites C
            if (!p->accumulate) {
                rest = p->tail.get();  // made by gern_gemm_create
                if (rest == nullptr) {
                    return fail("gern_gemm_run: the pipeline has no kernel for the last K % 4 columns");
                }
            }
            hip::MatrixF32 a2{a.data + k_main, M, K - k_main, K};
            hip::MatrixF32 b2{b.data + k_main * N, K - k_main, N, N};
            int64_t k_rest = K - k_main;
            rest->setStream(stream);
            rest->evaluate({{"A", &a2}, {"B", &b2}, {"C", &c}, {"k_dim", &k_rest}});
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    return 0;
}

int gern_qk_softmax_create(int64_t head_dim, int64_t max_keys, int flags, gern_pipeline *out) {
    if (out == nullptr) {
        return fail("gern_qk_softmax_create: null argument");
    }
    *out = nullptr;
    if (head_dim < 32 || head_dim > 256 || head_dim % 32 != 0) {
        return fail("gern_qk_softmax_create: head_dim must be a multiple of 32 in [32, 256]");
    }
    // The tile kernel holds one 256-column piece of a row per workgroup, whatever the row's width; the
    // row-block kernel keeps sixteen whole rows in the registers of one workgroup.
    const bool tiles = head_dim % 64 == 0 && !(flags & GERN_PIPELINE_QK_ROW_BLOCKS);
    if (max_keys < 256 || max_keys > (tiles ? GERN_QK_MAX_KEYS : 4096) || max_keys % 256 != 0) {
        return fail(tiles ? "gern_qk_softmax_create: max_keys must be a multiple of 256 in [256, GERN_QK_MAX_KEYS = 65536]"
                          : "gern_qk_softmax_create: max_keys must be a multiple of 256 in [256, 4096] for head dimensions that are not "
                            "multiples of 64 (and with GERN_PIPELINE_QK_ROW_BLOCKS)");
    }
    auto p = std::make_unique<gern_pipeline_s>();
    p->kind = gern_pipeline_s::QK_SOFTMAX;
    p->head_dim = head_dim;
    p->ncol = max_keys;
    p->qk_tiles = tiles;
    try {
        auto Q = AbstractDataTypePtr(new const annot::MatrixOperand("Q", annot::MatrixOperand::BF16));
        auto K = AbstractDataTypePtr(new const annot::MatrixOperand("K", annot::MatrixOperand::BF16));
        Variable rows("rows"), keys("keys"), d("d"), scale("scale", Datatype::Float32), threads("threads");
        Composable program;
        if (p->qk_tiles) {
            // 256 x 256 tiles of S, one per workgroup; column blocks along x so that the
            // workgroups of a row block, which wait for one another, have consecutive ids.
            using Tile256 = annot::ScoreTileF32;
            auto S = AbstractDataTypePtr(new const Tile256("S", Tile256::OUTPUT));
            auto logits = AbstractDataTypePtr(new const Tile256("logits", Tile256::TEMP));
            auto exchange = AbstractDataTypePtr(new const annot::RowStatsExchange("exchange"));
            annot::QKScaled qk{Q, K, logits};
            annot::SoftmaxAcrossTiles softmax{logits, exchange, S};
            program = Global((Tile(S["row"], rows.bind(256)) || Grid::BLOCK_Y)((Tile(S["col"], keys.bind(256)) || Grid::BLOCK_X)(
                                 qk[{{"d", d.bind(head_dim)}}](Q, K, logits, scale), softmax(logits, exchange, S))),
                             {{Grid::BLOCK_DIM_X, threads.bind(512)}});
        } else {
            auto S = AbstractDataTypePtr(new const annot::RowBlockF32("S", annot::RowBlockF32::OUTPUT));
            auto logits = AbstractDataTypePtr(new const annot::RowBlockF32("logits", annot::RowBlockF32::TEMP));
            auto shifted = AbstractDataTypePtr(new const annot::RowBlockF32("shifted", annot::RowBlockF32::TEMP));
            auto expd = AbstractDataTypePtr(new const annot::RowBlockF32("expd", annot::RowBlockF32::TEMP));
            auto row_max = AbstractDataTypePtr(new const annot::RowStat("row_max"));
            auto row_sum = AbstractDataTypePtr(new const annot::RowStat("row_sum"));
            annot::QKScaled qk{Q, K, logits};
            annot::MaxRow max_row{logits, row_max};
            annot::SubtractVec sub{row_max, logits, shifted};
            annot::ExpMatrix ex{shifted, expd};
            annot::SumRow sum_row{expd, row_sum};
            annot::DivideVecWholeRows div{row_sum, expd, S};
            std::map<std::string, Variable> width{{"ncol", keys.bind(max_keys)}};
            program = Global(
                (Tile(S["row"], rows.bind(16)) || Grid::BLOCK_X)(Tile(S["col"], keys.bind(max_keys))(
                    qk[{{"d", d.bind(head_dim)}}](Q, K, logits, scale), max_row[width](row_max, logits),
                    sub(row_max, logits, shifted), ex(shifted, expd), sum_row[width](row_sum, expd),
                    div(row_sum, expd, S))),
                // gernels/qk_softmax.h, qk_waves(): more wavefronts share a row
                // block as it gets wider.
                {{Grid::BLOCK_DIM_X, threads.bind(64 * qkWaves(max_keys))}});
        }
        // Tile kernel, rows of up to 4096 keys: XCD x takes row blocks x, x + 8, ... (bands of one row of tiles
        // dealt to the XCDs in turn), so the sixteen workgroups that exchange a row block's statistics and write
        // its rows sit on one XCD: 20.9 instead of 21.4-21.8 us at 4096 x 4096 x 128, same results.  A row block's
        // workgroups then lie within 8 x 16 = 128 consecutive launch numbers instead of 16, and that many must be
        // resident together for them to meet: taken only on a GPU with at least 256 CUs (one workgroup per CU), and
        // not for wider rows, whose row blocks would lie 8 x N / 256 launch numbers apart.
        bool rows_on_one_xcd = p->qk_tiles && max_keys <= 4096 && !(flags & GERN_PIPELINE_NO_XCD_REMAP);
        if (rows_on_one_xcd && !(flags & GERN_PIPELINE_COMPILE_ONLY)) {
            gern_hip_limits limits;
            rows_on_one_xcd = gern_hip_device_limits(&limits) == 0 && limits.compute_units >= 256;
        }
        if (experiments() && std::getenv("GERN_QK_PLAIN_ORDER") != nullptr) {
            rows_on_one_xcd = false;
        }
        int rc = rows_on_one_xcd ? finish(p.get(), program, flags, 0, 1) : finish(p.get(), program, flags | GERN_PIPELINE_NO_XCD_REMAP);
        if (rc != 0) {
            return rc;
        }
        if (p->qk_tiles && p->runner) {
            // Device memory of the exchange, all zeros (gernels/qk_tiles.h); owned by the pipeline.
            if (gern_hip_malloc(&p->qk_scratch, GERN_QK_SCRATCH_BYTES) != 0 ||
                gern_hip_memset(p->qk_scratch, 0, GERN_QK_SCRATCH_BYTES) != 0) {
                std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
                gern_hip_last_error(msg.data(), msg.size());
                return fail("gern_qk_softmax_create: " + msg);
            }
            // Look the library's own exchange memory up now (the runtime loads the library's code object at
            // the first lookup on a GPU), so that gern_qk_softmax_run_no_alloc never does.
            if (gern_detail_qk_shared_scratch != nullptr && gern_detail_qk_shared_scratch(&p->qk_shared_scratch) != 0) {
                return 1;  // message set
            }
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    *out = p.release();
    return 0;
}

namespace {

// Polls before a wavefront of the tile kernel gives up on the other tiles of its
// row block (a poll takes a microsecond or two); GERN_QK_SPIN_LIMIT, a whole
// number from 0 to 2^31 - 1, overrides it.  False: the variable holds something else.
bool qkSpinLimit(int32_t *limit) {
    *limit = 1 << 18;
    const char *forced = std::getenv("GERN_QK_SPIN_LIMIT");
    if (forced == nullptr) {
        return true;
    }
    char *end = nullptr;
    errno = 0;
    const long long v = std::strtoll(forced, &end, 10);
    if (end == forced || *end != '\0' || errno != 0 || v < 0 || v > 0x7FFFFFFFll) {
        return false;
    }
    *limit = (int32_t)v;
    return true;
}

}  // namespace

// Sets the calling thread's error message (for csrc/qk_no_alloc.hip).
__attribute__((visibility("hidden"))) int gern_detail_fail(const char *message) {
    return fail(message);
}

// One run of either QK program; `scratch` (tile program only) is
// GERN_QK_SCRATCH_BYTES of device memory that no other run uses at the same time.
// Internal to this library (shared with csrc/qk_no_alloc.hip).
__attribute__((visibility("hidden"))) int gern_detail_qk_softmax_run(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S, int64_t M, int64_t N,
                               float scale, void *scratch, void *stream, const char *who) {
    const std::string name(who);
    if (p == nullptr || p->kind != gern_pipeline_s::QK_SOFTMAX || Q == nullptr || K == nullptr || S == nullptr) {
        return fail(name + ": bad pipeline or null buffer");
    }
    if (!p->runner) {
        return fail(name + ": the pipeline was created compile-only");
    }
    if (M < 1 || N < 1 || N > p->ncol) {
        return fail(name + ": N exceeds the max_keys the pipeline was created for");
    }
    if (((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K)) & 15u) != 0 || (reinterpret_cast<uintptr_t>(S) & 3u) != 0) {
        return fail(name + ": Q and K are read in 16-byte pieces and must be 16-byte aligned (S 4-byte aligned)");
    }
    hip::MatrixF32 q{reinterpret_cast<float *>(const_cast<uint16_t *>(Q)), M, p->head_dim, p->head_dim};
    hip::MatrixF32 k{reinterpret_cast<float *>(const_cast<uint16_t *>(K)), N, p->head_dim, p->head_dim};
    hip::MatrixF32 s{S, M, N, N};
    try {
        p->runner->setStream(stream);
        p->last_stream = stream;
        if (!p->qk_tiles) {
            p->runner->evaluate({{"Q", &q}, {"K", &k}, {"S", &s}, {"scale", &scale}});
            return 0;
        }
        // entries: 8 bytes per (row of the padded row count, column block), sixteen column blocks per row
        const int64_t padded_rows = (M + 255) / 256 * 256;
        const int64_t pitch = ((N + 255) / 256 + 15) / 16 * 16;
        const int64_t capacity = ((int64_t)GERN_QK_SCRATCH_BYTES - 256) / 8;
        if (scratch == nullptr || padded_rows * pitch > capacity) {
            return fail(name + ": M x N needs more than GERN_QK_SCRATCH_BYTES of exchange memory (M up to 16384 at 4096 keys, "
                               "8192 at 8192, 1024 at 65536)");
        }
        int32_t spin_limit = 0;
        if (!qkSpinLimit(&spin_limit)) {
            return fail(name + ": GERN_QK_SPIN_LIMIT must be a whole number from 0 to 2147483647");
        }
        p->qk_used_shared = p->qk_used_shared || scratch != p->qk_scratch;
        annot::RowStatsExchangeLayout exchange{static_cast<char *>(scratch) + 256, scratch, (int32_t)pitch, spin_limit, capacity};
        p->runner->evaluate({{"Q", &q}, {"K", &k}, {"S", &s}, {"exchange", &exchange}, {"scale", &scale}});
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    return 0;
}

int gern_qk_softmax_run(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S, int64_t M, int64_t N,
                        float scale, void *stream) {
    return gern_detail_qk_softmax_run(p, Q, K, S, M, N, scale, p != nullptr ? p->qk_scratch : nullptr, stream,
                                      "gern_qk_softmax_run");
}

// The library's exchange memory as gern_qk_softmax_create found it for this pipeline (csrc/qk_no_alloc.hip
// calls this; it never looks anything up in a run).  Null with a message when the pipeline may not use it.
__attribute__((visibility("hidden"))) void *gern_detail_qk_shared_of(gern_pipeline p) {
    if (p == nullptr || p->kind != gern_pipeline_s::QK_SOFTMAX) {
        fail("gern_qk_softmax_run_no_alloc: bad pipeline");
        return nullptr;
    }
    if (p->qk_tiles && !p->qk_default_period) {
        // every user of the shared memory must agree on when the launch number wraps around
        fail("gern_qk_softmax_run_no_alloc: the pipeline was built with another GERN_QK_TAG_PERIOD than the library's exchange memory is used with");
        return nullptr;
    }
    if (p->qk_tiles && p->qk_shared_scratch == nullptr) {
        fail("gern_qk_softmax_run_no_alloc: the pipeline has no access to the library's exchange memory (created compile-only?)");
        return nullptr;
    }
    return p->qk_tiles ? p->qk_shared_scratch : static_cast<void *>(p);  // the other kernel needs none: any non-null value
}

int gern_pipeline_faults(gern_pipeline p, int64_t *count) {
    if (p == nullptr || count == nullptr) {
        return fail("gern_pipeline_faults: null argument");
    }
    *count = 0;
    try {
        for (Runner *r : {p->runner.get(), p->exact.get(), p->tail.get()}) {
            if (r != nullptr) {
                *count += r->ldsOverflows();  // waits for the device; zero for kernels without the LDS allocator
            }
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    if (!p->qk_tiles || !p->runner) {
        return 0;
    }
    if (gern_hip_sync() != 0) {
        std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
        gern_hip_last_error(msg.data(), msg.size());
        return fail("gern_pipeline_faults: " + msg);
    }
    // words 2 and 3 of the exchange's state: wavefronts that gave up, (row, column block) pairs that did not fit
    for (void *scratch : {p->qk_scratch, p->qk_used_shared ? p->qk_shared_scratch : nullptr}) {
        if (scratch == nullptr) {
            continue;
        }
        uint32_t words[2] = {0, 0};
        char *at = static_cast<char *>(scratch) + 8;
        if (gern_hip_memcpy_d2h(words, at, sizeof(words)) != 0 || ((words[0] | words[1]) != 0 && gern_hip_memset(at, 0, sizeof(words)) != 0)) {
            std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
            gern_hip_last_error(msg.data(), msg.size());
            return fail("gern_pipeline_faults: " + msg);
        }
        *count += (int64_t)words[0] + (int64_t)words[1];
    }
    p->qk_used_shared = false;
    return 0;
}

// User-level GEMM schedules over the LDS-staged matrices (annot/lds_matrix.h), as the reference's
// gernels/mm/kernel_3.cu, kernel_6.cu and kernel_10.cu compose them, sized for 64-lane wavefronts.
int gern_gemm_schedule_create(int schedule, int flags, gern_pipeline *out) {
    if (out == nullptr) {
        return fail("gern_gemm_schedule_create: null argument");
    }
    *out = nullptr;
    if (schedule != 3 && schedule != 6 && schedule != 10) {
        return fail("gern_gemm_schedule_create: schedule must be 3, 6 or 10 (the reference's gernels/mm/kernel_<n>.cu)");
    }
    constexpr int N = GERN_GEMM_SCHEDULE_SIZE;
    auto p = std::make_unique<gern_pipeline_s>();
    p->kind = gern_pipeline_s::GEMM_SCHEDULE;
    try {
        using CType = annot::MatrixGlobalToGlobal<N, N>;
        // a staged copy of C is written back only if the data structure says its queries are copies
        struct CWrittenBack : CType {
            using CType::CType;
            bool insertQuery() const override {
                return true;
            }
        };
        AbstractDataTypePtr A, B;
        AbstractDataTypePtr C(schedule != 3 ? static_cast<const AbstractDataType *>(new const CWrittenBack("C", false))
                                             : static_cast<const AbstractDataType *>(new const CType("C", false)));
        if (schedule == 3) {
            A = AbstractDataTypePtr(new const annot::MatrixGlobalToShared<N, N>("A", false));
            B = AbstractDataTypePtr(new const annot::MatrixGlobalToShared<N, N>("B", false));
        } else if (schedule == 6) {
            A = AbstractDataTypePtr(new const annot::MatrixGlobalToSharedVec<N, N>("A", false));
            B = AbstractDataTypePtr(new const annot::MatrixGlobalToSharedVec<N, N>("B", false));
        } else {
            A = AbstractDataTypePtr(new const annot::MatrixGlobalToSharedFlat<N, N>("A", false));
            B = AbstractDataTypePtr(new const annot::MatrixGlobalToSharedFlat<N, N>("B", false));
        }
        annot::MatrixGlobalToShared<N, N> view_of("A_view", false);
        annot::MatrixQueryRegNoVector<N, N> in_registers("C_reg", false);
        Variable k_dim("k_dim"), k_tiled("k_tiled"), block_x("block_x"), block_y("block_y"), thread_x("thread_x"), thread_y("thread_y"),
            thread_k("thread_k"), warp_x("warp_x"), warp_y("warp_y"), lanes_y("lanes_y"), one_val("one_val"), smem_size("smem_size");
        k_dim = k_dim.bind(N);
        annot::MatrixMultiplyScalar mm(A, B, C);
        auto &mm_sp = mm[{{"k_dim", k_dim}}];
        Composable program;
        if (schedule == 10) {
            // kernel_10.cu:108-131: block tile -> wavefront tile -> one output per lane, register copies of C, A and B.
            // K tiles of 32: a lane then holds 32 + 32 operand values, within the 128 registers that a
            // workgroup of 1024 threads leaves each lane (64-deep tiles spill to scratch memory).
            int64_t kt10 = 32;
            if (const char *v = std::getenv("GERN_SCHEDULE_TILES"); v != nullptr && experiments()) {
                kt10 = std::atoll(v);
            }
            Composable per_lane = Stage(
                C, in_registers.getQueryFunction(), in_registers.getInsertFunction(),
                Stage(A, in_registers.getQueryFunction(),
                      Stage(B, in_registers.getQueryFunction(),
                            Reduce(k_dim, thread_k.bind(8))(Stage(A, view_of.getView(), Stage(B, view_of.getView(), mm_sp(A, B, C)))))));
            // The lanes of a wavefront (64 consecutive threadIdx.x) take 64 consecutive COLUMNS of one row of C:
            // they then read the same element of the staged A tile (one LDS access, broadcast), consecutive
            // elements of the staged B tile (all banks) and write consecutive floats of C.  kernel_10.cu puts
            // consecutive lanes on consecutive rows; on the dense tiles that direct loads leave in LDS that makes
            // every lane of a read hit the same bank (measured: 2064 us at 1024^3 against the time below).
            const bool rows_on_lanes = std::getenv("GERN_SCHEDULE_ROWS_ON_LANES") != nullptr && experiments();
            if (rows_on_lanes) {
                Composable lanes = (Tile(C["row"], thread_x.bind(1)) || Grid::Unit::THREAD_X_IN_WRAPS)(
                    (Tile(C["col"], thread_y.bind(1)) || Grid::Unit::THREAD_Y_IN_WRAPS)(per_lane));
                Composable waves =
                    (Tile(C["row"], warp_x.bind(64)) || Grid::Unit::WARP_Y)((Tile(C["col"], warp_y.bind(16)) || Grid::Unit::WARP_X)(lanes));
                program = Global((Tile(C["row"], block_x.bind(64)) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y.bind(16)) || Grid::Unit::BLOCK_Y)(
                                     Reduce(k_dim, k_tiled.bind(kt10))(Stage(A, Stage(B, waves))))),
                                 {{Grid::Dim::BLOCK_DIM_Y, lanes_y.bind(16)}}, smem_size, annot::LdsManager(smem_size));
            } else {
                Composable lanes = (Tile(C["col"], thread_y.bind(1)) || Grid::Unit::THREAD_X_IN_WRAPS)(
                    (Tile(C["row"], thread_x.bind(1)) || Grid::Unit::THREAD_Y_IN_WRAPS)(per_lane));
                Composable waves =
                    (Tile(C["col"], warp_y.bind(64)) || Grid::Unit::WARP_Y)((Tile(C["row"], warp_x.bind(16)) || Grid::Unit::WARP_X)(lanes));
                program = Global((Tile(C["col"], block_y.bind(64)) || Grid::Unit::BLOCK_X)((Tile(C["row"], block_x.bind(16)) || Grid::Unit::BLOCK_Y)(
                                     Reduce(k_dim, k_tiled.bind(kt10))(Stage(A, Stage(B, waves))))),
                                 {{Grid::Dim::BLOCK_DIM_Y, lanes_y.bind(16)}}, smem_size, annot::LdsManager(smem_size));
            }
        } else if (schedule == 6) {
            // The composition of kernel_6.cu:61-74 (block tile staged through LDS 16 bytes per lane, thread
            // tiles, windows of the staged tiles per thread) with one more Stage: the thread's tile of C is
            // copied into registers.  That copy does not depend on the loop over K tiles, so the lowering
            // makes it before the loop and writes it back after it, and matrix_multiply runs on a register
            // tile (the reference's composition multiplies into C in global memory, a load and a store per
            // term).  64 x 64 block tiles and 4 x 4 outputs per thread make workgroups of four wavefronts and
            // 256 workgroups at 1024^2: one per compute unit.
            int64_t bm = 64, bn = 64, kt = 64, tm = 4, tn = 4;
            if (const char *v = std::getenv("GERN_SCHEDULE_TILES"); v != nullptr && experiments()) {
                long long a[5] = {bm, bn, kt, tm, tn};
                std::sscanf(v, "%lld,%lld,%lld,%lld,%lld", &a[0], &a[1], &a[2], &a[3], &a[4]);
                bm = a[0], bn = a[1], kt = a[2], tm = a[3], tn = a[4];
            }
            Composable per_thread = Stage(C, in_registers.getQueryFunction(), in_registers.getInsertFunction(),
                                          Stage(A, view_of.getViewVec(), Stage(B, view_of.getViewVec(), mm_sp(A, B, C))));
            program = Global((Tile(C["row"], block_x.bind(bm)) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y.bind(bn)) || Grid::Unit::BLOCK_Y)(
                                 Reduce(k_dim, k_tiled.bind(kt))(Stage(A, Stage(B, (Tile(C["row"], thread_x.bind(tm)) || Grid::Unit::THREAD_Y)(
                                                                                       (Tile(C["col"], thread_y.bind(tn)) || Grid::Unit::THREAD_X)(per_thread))))))),
                             {}, smem_size, annot::LdsManager(smem_size));
        } else {
            // kernel_3.cu:61-75: block tile staged through LDS one float per lane, 4 x 4 outputs per thread multiplied
            // straight into C in global memory; 64 x 64 block tiles make workgroups of 256 threads
            Composable inner = Reduce(k_dim, one_val.bind(16))(Stage(A, view_of.getView(), Stage(B, view_of.getView(), mm_sp(A, B, C))));
            program = Global((Tile(C["row"], block_x.bind(64)) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y.bind(64)) || Grid::Unit::BLOCK_Y)(
                                 Reduce(k_dim, k_tiled.bind(16))(Stage(A, Stage(B, (Tile(C["row"], thread_x.bind(4)) || Grid::Unit::THREAD_Y)(
                                                                                       (Tile(C["col"], thread_y.bind(4)) || Grid::Unit::THREAD_X)(inner))))))),
                             {}, smem_size, annot::LdsManager(smem_size));
        }
        int rc = finish(p.get(), program, flags | GERN_PIPELINE_NO_XCD_REMAP);
        if (rc != 0) {
            return rc;
        }
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    *out = p.release();
    return 0;
}

int gern_gemm_schedule_run(gern_pipeline p, const float *A, const float *B, float *C, void *stream) {
    if (p == nullptr || p->kind != gern_pipeline_s::GEMM_SCHEDULE || A == nullptr || B == nullptr || C == nullptr) {
        return fail("gern_gemm_schedule_run: bad pipeline or null buffer");
    }
    if (!p->runner) {
        return fail("gern_gemm_schedule_run: the pipeline was created compile-only");
    }
    hip::GlobalMatrixF32 a{const_cast<float *>(A)}, b{const_cast<float *>(B)}, c{C};
    int64_t smem = 48 * 1024;
    if (const char *v = std::getenv("GERN_SCHEDULE_LDS_KB"); v != nullptr && experiments()) {
        smem = std::atoll(v) * 1024;
    }
    try {
        p->runner->setStream(stream);
        p->runner->evaluate({{"A", &a}, {"B", &b}, {"C", &c}, {"smem_size", &smem}});
    } catch (const std::exception &e) {
        return fail(e.what());
    }
    return 0;
}

const char *gern_pipeline_source(gern_pipeline p) {
    if (p == nullptr) {
        return "";
    }
    return p->last_run_exact && !p->exact_source.empty() ? p->exact_source.c_str() : p->source.c_str();
}

const char *gern_pipeline_kernel_name(gern_pipeline p) {
    if (p == nullptr) {
        return "";
    }
    if (p->kernel_name.empty() && p->runner) {
        p->kernel_name = p->runner->getKernelName();
    }
    if (p->last_run_exact && !p->exact_kernel_name.empty()) {
        return p->exact_kernel_name.c_str();
    }
    return p->kernel_name.c_str();
}

int gern_pipeline_destroy(gern_pipeline p) {
    if (p != nullptr) {
        // waits for the device, then frees the loaded code objects
        for (Runner *r : {p->runner.get(), p->exact.get(), p->tail.get()}) {
            if (r != nullptr) {
                r->release();
            }
        }
        if (p->qk_scratch != nullptr) {
            gern_hip_free(p->qk_scratch);
        }
    }
    delete p;
    return 0;
}

size_t gern_pipelines_last_error(char *buf, size_t buf_size) {
    if (buf != nullptr && buf_size > 0) {
        size_t n = g_error.size() < buf_size - 1 ? g_error.size() : buf_size - 1;
        std::memcpy(buf, g_error.data(), n);
        buf[n] = '\0';
    }
    return g_error.size();
}

}  // extern "C"
