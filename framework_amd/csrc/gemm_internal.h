// Launch descriptors shared by the GEMM kernels and their dispatcher.
#pragma once
#include <stdint.h>

namespace mni {

// Everything a GEMM kernel needs, passed by value as the kernel argument.
// op(A)[b](m, k) = A[(b % a_bcount) * a_bs + m * a_rs + k * a_cs]
// op(B)[b](k, n) = B[(b % b_bcount) * b_bs + k * b_rs + n * b_cs]
struct GemmLaunch {
    const float *A;
    const float *B;
    float *C;
    const float *bias;
    // One pointer, three mutually exclusive uses (a fourth 64-byte line of kernel
    // arguments would cost every launch a further scalar fetch): the split-K /
    // stream-K partials; with MNI_EPI_BIAS_GELU_DUAL the second output
    // gelu(C + bias), laid out like C; with MNI_EPI_DGELU the saved
    // pre-activation z (C then becomes acc * gelu'(z + bias)), laid out like C.
    union {
        float *ws;  // split-K partials [slice][batch][M][N]
        float *aux_out;
        const float *aux_in;
    };
    int M, N, K, batch;
    int64_t a_rs, a_cs, a_bs;
    int64_t b_rs, b_cs, b_bs;
    int a_bcount, b_bcount;
    int64_t ldc, c_bs;
    int split_k, k_per_slice;
    int tiles_m, tiles_n;
    int epilogue, accumulate;
    // Stream-K form (streamk != 0, split_k == 1): the grid is xcds * sk_wpx
    // persistent workgroups; `ws` then holds one tile-sized partial per
    // workgroup and sk_flags one arrival mark per workgroup, set to sk_epoch.
    int streamk, sk_wpx, sk_xcds;
    // stream-K arrival marks; with MNI_EPI_DGELU (never stream-K) the column sums
    // of C per 64-row (32-row for 64-row tiles) strip, [batch][2 tiles_m][N], or null
    union {
        unsigned *sk_flags;
        float *colsum_part;
    };
    unsigned sk_epoch;
    unsigned *status;  // device status word: set when a finisher's bounded wait expires
};

// tile_m, tile_n in {128, 64}; g.tiles_m / g.tiles_n count tiles of that size
int launch_gemm_mfma(const GemmLaunch &g, int amode, int bmode, int tile_m, int tile_n);
// Column sums of a contiguous [rows, cols] matrix that a paired launch computes along with its two products (in the
// tiny-product pair: rows added in order; in the tile kernel's pair: in 64 interleaved groups of rows, the groups then
// added in order); `done` says whether the launch did.
struct PairColsum {
    const float *src;
    float *out;
    int64_t rows, cols;
    bool done;
};
// Two independent products, both of 64 x 64 or both of 128 x 128 tiles (`tile`; one workgroup per tile, all of K) in one
// launch; amode0 must be 0 and bmode1 1.
bool gemm_mfma_pair_eligible(int amode0, int bmode0, int amode1, int bmode1);
// `colsum` (may be null): column sums computed by extra workgroups of the same launch; must satisfy gemm_mfma_pair_takes_colsum.
bool gemm_mfma_pair_takes_colsum(const PairColsum &cs);
int launch_gemm_mfma_pair(const GemmLaunch &g0, int amode0, int bmode0, const GemmLaunch &g1, int amode1, int bmode1, int tile,
                          const PairColsum *colsum = nullptr);
// workgroups that stay resident per CU for a tile shape (what the stream-K grid is sized by)
int gemm_mfma_resident_per_cu(int tile_m, int tile_n);
int gemm_mfma_tile_k();
// Register-direct form for batched products of many small tiles (gemm_direct.hip):
// 64 x 64 tiles (g.tiles_m / g.tiles_n count those), one wavefront per tile
// (ksplit 1) or four wavefronts sharing K (ksplit 4).  amode / bmode as for
// the tile kernel; both must be 0 or 1 and pass gemm_direct_eligible.
bool gemm_direct_eligible(const GemmLaunch &g, int amode, int bmode);
int launch_gemm_direct(const GemmLaunch &g, int amode, int bmode, int ksplit);
// One thread per output, sequential K (gemm_tiny.hip): a few thousand outputs of a short K, any strides.
bool gemm_tiny_eligible(const GemmLaunch &g);
int launch_gemm_tiny(const GemmLaunch &g);
int launch_gemm_tiny_pair(const GemmLaunch &g0, const GemmLaunch &g1, const PairColsum *colsum = nullptr);  // two eligible, independent products in one launch
// 9 to 32 rows of a K-contiguous A against a wide N-contiguous B, both straight into MFMA registers (gemm_fewrows.hip):
// g.tiles_n counts column groups of 128, g.split_k K slices of g.k_per_slice (a multiple of 32).  With split_k > 1:
// partials [slice][batch][M][N] in g.ws and one counter per (batch, column group) in g.sk_flags, zero between launches
// (the workgroup that completes a count adds the slices up and returns the counter to zero).
bool gemm_fewrows_eligible(const GemmLaunch &g, int amode, int bmode);
int launch_gemm_fewrows(const GemmLaunch &g, int amode, int bmode);
// Short-K form for an A contiguous along M and a B contiguous along N (gemm_outer.hip): K <= 512 outer products,
// both operands straight into MFMA registers, no epilogue; g.accumulate honoured.
bool gemm_outer_eligible(const GemmLaunch &g);
int launch_gemm_outer(const GemmLaunch &g);
// Short-K form for two K-contiguous operands (gemm_panel.hip): 128 x 128 tiles
// (g.tiles_m / g.tiles_n count those), all of K <= 64 at once.
bool gemm_panel_eligible(const GemmLaunch &g, int amode, int bmode);
int launch_gemm_panel(const GemmLaunch &g, int amode, int bmode);

// Skinny (GEMV-shaped) products: X (MR x K, MR <= 16) against a large W.
//   out[b](i, j) = sum_k X[b](i, k) * W[b](k, j),  i < rows, j < cols
// written at out[b * o_bs + i * o_rs + j * o_cs] (or to split-K partials).
struct SkinnyLaunch {
    const float *X;
    const float *W;
    float *out;
    const float *bias;  // indexed by bias_on_rows ? i : j
    float *ws;          // partials [slice][batch][rows][pitch]: pitch = cols, or, in the single-launch form, cols
                        // rounded up to whole 128-byte lines (skinny_ws_pitch), so that no line is shared by two units
    int rows, cols, K, batch;
    int groups;  // column groups of skinny_cols_block_cols() (skinny_cols only)
    int64_t x_rs, x_cs, x_bs;  // X(i, k)
    int64_t w_rs, w_cs, w_bs;  // W(k, j)
    int x_bcount, w_bcount;
    int64_t o_rs, o_cs, o_bs;
    int split_k, k_per_slice;
    int epilogue, accumulate, bias_on_rows;
    // Single-launch form (split_k > 1): arrival flags [unit][split_k] with
    // unit = b * groups + column group, and the value that marks this launch.
    // (The struct is the kernel argument: it is kept to three 64-byte lines,
    // a fourth costs the kernel's start a further scalar fetch.)
    unsigned *flags;
    unsigned epoch;
    // Single-launch form: at most this many workgroups per unit add up its slices (each then takes every
    // max_reducers-th row).  Reducers hold their places while they wait, so all of an XCD's must fit on it at once.
    int max_reducers;
    unsigned *status;  // device status word: set when a reducer's bounded wait expires
};
// W with unit stride along j (cols): lanes own columns, K split over wavefronts and slices.
// xcds > 0: the single-launch form, units dealt over that many XCDs; 0: partials left for a reduction launch.
int launch_skinny_cols(const SkinnyLaunch &s, int xcds);
// workgroups of the single-launch form of `s` that fit one CU together (0: unknown)
int skinny_cols_fused_occupancy(const SkinnyLaunch &s);
// floats per row of the K-slice partials
int skinny_ws_pitch(int cols, bool single_launch);
// W with unit stride along k: one wavefront per output column, shuffle reduce.
int launch_skinny_dots(const SkinnyLaunch &s);
int skinny_cols_block_cols();
int skinny_cols_rows_per_pass();  // K rows one workgroup covers per trip

// The decode product (gemm_gemv.hip): up to 8 rows of a K-contiguous X against a row-major W, one workgroup of 16
// wavefronts per CU; workgroup id -> (unit = id % units: 128 columns, slice = id / units: trips * 512 rows of K).
// Partials carry the launch's tag (epoch) in every piece; pa / pb / count belong to the library (DeviceCtx) and are
// written by nothing else.
static constexpr int GEMV_MAX_SLICES = 8;
static constexpr int GEMV_COUNTERS_PER_UNIT = 4;  // one per summing wavefront (rows * 32 threads)
struct GemvLaunch {
    const float *W;
    const float *X;
    float *out;
    const float *bias;  // one value per column, 16-byte aligned, or null
    float __attribute__((ext_vector_type(4))) *pa;  // [unit][slice][rows * 32] pieces {x, y, z, tag}
    float __attribute__((ext_vector_type(2))) *pb;  // the same of {w, tag}
    unsigned *count;   // [unit][GEMV_COUNTERS_PER_UNIT], zero between launches (each count wraps to zero with its last arrival)
    unsigned *status;  // device status word: set when the adding wavefront's bounded wait for a partial expires
    unsigned epoch;
    int units, slices, trips;
    int w_rs, x_rs, o_rs;
    int epilogue, accumulate;
    int rows;  // (the 16-row form: rows of X that exist; the forms up to 8 rows are compiled per row count)
};
// Whether the kernel takes rows x K against K x cols on this device, and with how many K slices / trips per workgroup.
bool gemv_units_plan(int rows, int cols, int K, int cus, int xcds, int *slices, int *trips);
size_t gemv_units_partial_slots(int rows, int cols, int slices);  // pieces of pa (and of pb) the plan writes
int launch_gemv_units(const GemvLaunch &p, int rows);
// The same for up to 32 rows (two sets of 16): units of 64 columns, 1024 rows of K per workgroup and trip.
bool gemv_units16_plan(int rows, int cols, int K, int cus, int xcds, int *slices, int *trips);
size_t gemv_units16_partial_slots(int rows, int cols, int slices);
bool gemv_units16_pitches_ok(int64_t w_rs, int64_t x_rs);  // the kernel's 32-bit byte offsets hold for these pitches
size_t gemv_units16_counters(int rows, int cols);  // counters the plan uses (one per summing wavefront and unit)
int launch_gemv_units16(const GemvLaunch &p);

// Up to 32 rows against a wide K-contiguous operand (gemm_fewrows_nt.hip): a wavefront per 16 columns and all of K, A in LDS.
static constexpr int FEWROWS_NT_LDS_FLOATS = 33024;  // 4, 8, 16 or 32 rows of K + 16 floats: 8 rows of 4096, 16 of 2048
struct FewNtLaunch {
    const float *X;     // [M, K], rows x_rs apart
    const float *W;     // [N, K], rows w_cs apart
    float *out;         // [M, N], rows o_rs apart
    const float *bias;  // one value per column, or null
    int M, N, K;
    int64_t x_rs, w_cs, o_rs;
    int epilogue, accumulate;
    // the form with K in slices only (null / zero otherwise):
    float *ws;        // partial sums [column block of 64][slice][column 64][row 16]
    unsigned *count;  // one counter per column block, zero between launches (each wraps to zero with its last arrival)
    int slices;       // K slices: runs of K's steps of 64 values, the first ksteps % slices of them one step longer
    int ksteps;       // K / 64
};
bool gemm_fewrows_nt_eligible(const GemmLaunch &g, int amode, int bmode);
int launch_gemm_fewrows_nt(const GemmLaunch &g, int amode, int bmode);
// The same product with K beyond what LDS holds of A, or too few columns to give every CU a workgroup: K in slices
// (workgroup = 64 columns x one slice), the slices of a column block added up by the last of them to arrive.
static constexpr int FEWROWS_NT_MAX_SLICES = 16;
bool gemm_fewrows_nt_sliced_eligible(const GemmLaunch &g, int amode, int bmode);
int fewrows_nt_max_steps(int rows);  // steps of 64 values of K a slice may have with that many rows of A
size_t fewrows_nt_sliced_ws_floats(int N, int slices);
int launch_gemm_fewrows_nt_sliced(const GemmLaunch &g, int amode, int bmode, int slices, float *ws, unsigned *count);

// Sums split-K partials ws[slice][batch][rows][cols] in slice order and
// applies the epilogue; out addressed with (o_bs, o_rs, o_cs).
struct ReduceLaunch {
    const float *ws;
    float *out;
    const float *bias;
    int slices, batch, rows, cols;
    int64_t o_rs, o_cs, o_bs;
    int epilogue, accumulate, bias_on_rows;
};
int launch_splitk_reduce(const ReduceLaunch &r);
int launch_skinny_reduce(const ReduceLaunch &r);  // few outputs, many slices

}  // namespace mni
