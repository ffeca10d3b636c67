// mni_rocm_sgemm: validation, kernel choice (MFMA tile kernel vs the skinny
// bandwidth kernels), operand-layout classification and the split-K plan.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// 0: K axis contiguous, 1: the other axis contiguous, 2: arbitrary.  `ks` is
// the stride along K, `os` the stride along M (for A) or N (for B).  Base
// address, leading dimension and batch stride do not matter: the tile kernel's
// 16-byte loads work from any 4-byte aligned address.
static int classify(int64_t ks, int64_t os) {
    if (ks == 1) return 0;
    if (os == 1) return 1;
    return 2;
}

static int validate(const mni_gemm_desc &d) {
    if (d.M < 0 || d.N < 0 || d.K < 0 || d.batch < 0)
        return set_error(MNI_ERR_INVALID, "sgemm: negative extent (M=%lld N=%lld K=%lld batch=%lld)",
                         (long long)d.M, (long long)d.N, (long long)d.K, (long long)d.batch);
    if (d.M > 0x7fffffffLL || d.N > 0x7fffffffLL || d.K > 0x7fffffffLL || d.batch > 0x7fffffffLL)
        return set_error(MNI_ERR_INVALID, "sgemm: extent exceeds 2^31-1");
    if (d.M == 0 || d.N == 0 || d.batch == 0) return MNI_OK;
    if (!d.C) return set_error(MNI_ERR_INVALID, "sgemm: C is null");
    if (d.K > 0 && (!d.A.ptr || !d.B.ptr)) return set_error(MNI_ERR_INVALID, "sgemm: operand pointer is null");
    if (d.A.batch_count < 1 || d.B.batch_count < 1)
        return set_error(MNI_ERR_INVALID, "sgemm: operand batch_count must be >= 1");
    if (d.ldc < d.N) return set_error(MNI_ERR_INVALID, "sgemm: ldc (%lld) < N (%lld)", (long long)d.ldc, (long long)d.N);
    if (d.epilogue < MNI_EPI_NONE || d.epilogue > MNI_EPI_DGELU)
        return set_error(MNI_ERR_INVALID, "sgemm: unknown epilogue %d", d.epilogue);
    if (d.epilogue >= MNI_EPI_BIAS_GELU_DUAL) {
        if (!d.aux) return set_error(MNI_ERR_INVALID, "sgemm: epilogue %d needs the aux pointer", d.epilogue);
        if (d.accumulate || d.split_k > 1)
            return set_error(MNI_ERR_INVALID, "sgemm: epilogue %d takes neither accumulate nor split_k", d.epilogue);
        if (d.algo != MNI_ALGO_AUTO && d.algo != MNI_ALGO_MFMA && d.algo != MNI_ALGO_MFMA_SMALL)
            return set_error(MNI_ERR_INVALID, "sgemm: epilogue %d runs on the MFMA tile kernel only", d.epilogue);
    }
    if (d.colsum_part && d.epilogue != MNI_EPI_DGELU)
        return set_error(MNI_ERR_INVALID, "sgemm: colsum_part goes with the DGELU epilogue only");
    if (d.epilogue != MNI_EPI_NONE && !d.bias)
        return set_error(MNI_ERR_INVALID, "sgemm: epilogue %d needs a bias pointer", d.epilogue);
    if (d.split_k < 0) return set_error(MNI_ERR_INVALID, "sgemm: split_k < 0");
    if (d.algo < MNI_ALGO_AUTO || d.algo > MNI_ALGO_FEWROWS_NT)
        return set_error(MNI_ERR_INVALID, "sgemm: unknown algo %d", d.algo);
    return MNI_OK;
}

static int finish_split(const float *ws, float *out, const float *bias, int slices, int batch, int rows, int cols,
                        int64_t o_rs, int64_t o_cs, int64_t o_bs, int epilogue, int accumulate, int bias_on_rows) {
    ReduceLaunch r;
    r.ws = ws; r.out = out; r.bias = bias;
    r.slices = slices; r.batch = batch; r.rows = rows; r.cols = cols;
    r.o_rs = o_rs; r.o_cs = o_cs; r.o_bs = o_bs;
    r.epilogue = epilogue; r.accumulate = accumulate; r.bias_on_rows = bias_on_rows;
    return launch_splitk_reduce(r);
}

// A fresh value for the arrival marks of a single-launch reduction (skinny
// fused kernel, stream-K): marks from earlier launches never match it, so the
// array needs no clearing except when the counter wraps.
static int next_epoch(unsigned *epoch) {
    DeviceCtx &c = ctx();
    if (++c.skinny_epoch == 0) {
        MNI_TRY(k_fill((float *)c.skinny_flags, 0.0f, (int64_t)c.skinny_flag_cap));
        MNI_TRY(k_fill((float *)c.gemv_pa, 0.0f, (int64_t)c.gemv_slot_cap * 4));  // (the decode product's tags are epochs too)
        MNI_TRY(k_fill((float *)c.gemv_pb, 0.0f, (int64_t)c.gemv_slot_cap * 2));
        c.skinny_epoch = 1;
    }
    *epoch = c.skinny_epoch;
    return MNI_OK;
}

// ---- the decode product ---------------------------------------------------------
// x[<= 32, K] against a row-major W[K, N] whose column and K extents deal the CUs one workgroup each (gemm_gemv.hip).
// True when it took the product (errors through *rc).
static bool try_gemv_units(const SkinnyLaunch &s, const mni_gemm_desc &d, int *rc) {
    DeviceCtx &c = ctx();
    if (d.algo != MNI_ALGO_AUTO && d.algo != MNI_ALGO_GEMV) return false;
    if (d.split_k > 1 || s.batch != 1 || s.rows > 32 || s.x_cs != 1 || s.w_cs != 1 || s.o_cs != 1) return false;
    if ((s.w_rs % 4) != 0 || !aligned16(s.W) || (s.o_rs % 4) != 0 || !aligned16(s.out)) return false;
    if (s.w_rs > 0x7fffffffLL || s.x_rs > 0x7fffffffLL || s.o_rs > 0x7fffffffLL) return false;
    if (s.epilogue > MNI_EPI_BIAS_GELU || s.bias_on_rows) return false;
    if (s.epilogue != MNI_EPI_NONE && !aligned16(s.bias)) return false;
    if (s.accumulate && s.epilogue >= MNI_EPI_BIAS_RELU) return false;  // (the old output would have to wait for the sum)
    // Two forms.  Up to 8 rows on 4 x 4 x 1 blocks (128-column units, a kernel per row count); up to 32 rows on the
    // 16 x 16 x 4 MFMA (64-column units, X in 16-byte pieces, one or two sets of 16 rows), whose time depends on the number
    // of sets only.  Measured on MI355X, us, cold W, the first against the second: 4096 x 4096 1 row 12.2 / 13.7,
    // 4 rows 12.8 / 13.8, 6 rows 13.5 / 13.8, 7 rows 14.3 / 13.8, 8 rows 14.5 / 13.8 (16 rows 14.1: 20.9 through the
    // few-rows kernel); 8192 x 8192 4 rows 51.2 / 42.4 (the column kernel 45.0), 8 rows 52.4 / 43.0; 16384 x 1024 4 rows
    // 13.3 / 12.4, 8 rows 15.0 / 12.6; 4096 x 8192 4 rows 23.1 / 23.8, 8 rows 24.9 / 24.0.
    int slices = 0, trips = 0, slices16 = 0, trips16 = 0;
    const bool narrow_ok = s.rows <= 8 && c.gemv_pa && gemv_units_plan(s.rows, s.cols, s.K, c.compute_units, c.xcd_count, &slices, &trips) &&
                           gemv_units_partial_slots(s.rows, s.cols, slices) <= c.gemv_slot_cap &&
                           (size_t)(s.cols / 128) * GEMV_COUNTERS_PER_UNIT <= c.gemv_counter_cap;
    const bool wide_ok = c.gemv_pa && (s.x_rs % 4) == 0 && aligned16(s.X) && gemv_units16_pitches_ok(s.w_rs, s.x_rs) &&
                         gemv_units16_plan(s.rows, s.cols, s.K, c.compute_units, c.xcd_count, &slices16, &trips16) &&
                         gemv_units16_partial_slots(s.rows, s.cols, slices16) <= c.gemv_slot_cap &&
                         gemv_units16_counters(s.rows, s.cols) <= c.gemv_counter_cap;
    // Two sets of rows, us against the few-rows MFMA kernel (cold W of normally distributed values): 32 x 4096 x 4096 16.4 / 21.5,
    // 24 rows 16.1 / 21.4, 32 x 8192 x 4096 28.2 / 30.8, 32 x 4096 x 8192 28.3 / 33.9, 32 x 8192 x 8192 52.4 / 52.6, 24 rows 50.0 / 52.6,
    // 32 x 4096 x 16384 52.3 / 55.5, 32 x 16384 x 4096 50.2 / 52.2: taken wherever it is eligible.
    const bool prefer_wide = s.rows > 6 || s.cols > 4096;
    const bool wide = wide_ok && (prefer_wide || !narrow_ok);
    if (!wide && !narrow_ok) return false;
    if (wide) {
        slices = slices16;
        trips = trips16;
    } else if (d.algo == MNI_ALGO_AUTO && trips > 1 && s.cols > 4096) {
        // (several trips of the narrow form beyond 4096 columns: the column kernel's four small workgroups per CU are
        // ahead, 4 x 8192 x 8192 52.0 against 45.0; reached only where the wide form cannot take the product)
        return false;
    }
    GemvLaunch g;
    g.W = s.W; g.X = s.X; g.out = s.out; g.bias = s.bias;
    g.pa = (decltype(g.pa))c.gemv_pa; g.pb = (decltype(g.pb))c.gemv_pb;
    g.count = c.gemv_counters; g.status = c.status_dev;
    g.units = s.cols / (wide ? 64 : 128); g.slices = slices; g.trips = trips;
    g.w_rs = (int)s.w_rs; g.x_rs = (int)s.x_rs; g.o_rs = (int)s.o_rs;
    g.epilogue = s.epilogue; g.accumulate = s.accumulate; g.rows = s.rows;
    *rc = next_epoch(&g.epoch);
    if (*rc == MNI_OK) *rc = wide ? launch_gemv_units16(g) : launch_gemv_units(g, s.rows);
    return true;
}

// ---- skinny path --------------------------------------------------------------
// Returns 1 when it handled the product, 0 when the shape/layout is not
// eligible, < 0 ... never; errors are returned through *rc.
static bool try_skinny(const mni_gemm_desc &d, int *rc) {
    *rc = MNI_OK;
    if (d.K == 0) return false;
    SkinnyLaunch s;
    bool swapped;
    if (d.M <= 16) swapped = false;
    else if (d.N <= 16) swapped = true;
    else return false;

    for (int attempt = 0; attempt < 2; ++attempt) {
        if (!swapped) {
            s.rows = (int)d.M; s.cols = (int)d.N;
            s.X = d.A.ptr; s.x_rs = d.A.row_stride; s.x_cs = d.A.col_stride;
            s.x_bs = d.A.batch_stride; s.x_bcount = (int)d.A.batch_count;
            s.W = d.B.ptr; s.w_rs = d.B.row_stride; s.w_cs = d.B.col_stride;
            s.w_bs = d.B.batch_stride; s.w_bcount = (int)d.B.batch_count;
            s.o_rs = d.ldc; s.o_cs = 1; s.bias_on_rows = 0;
        } else {
            // C^T = B^T * A^T: the few columns of C become the rows of X.
            s.rows = (int)d.N; s.cols = (int)d.M;
            s.X = d.B.ptr; s.x_rs = d.B.col_stride; s.x_cs = d.B.row_stride;
            s.x_bs = d.B.batch_stride; s.x_bcount = (int)d.B.batch_count;
            s.W = d.A.ptr; s.w_rs = d.A.col_stride; s.w_cs = d.A.row_stride;
            s.w_bs = d.A.batch_stride; s.w_bcount = (int)d.A.batch_count;
            s.o_rs = 1; s.o_cs = d.ldc; s.bias_on_rows = 1;
        }
        s.K = (int)d.K; s.batch = (int)d.batch;
        s.out = d.C; s.o_bs = d.c_batch_stride; s.bias = d.bias;
        s.epilogue = d.epilogue; s.accumulate = d.accumulate;
        s.ws = nullptr; s.split_k = 1; s.k_per_slice = s.K;
        s.groups = 0; s.flags = nullptr; s.epoch = 0; s.max_reducers = 16; s.status = ctx().status_dev;

        if (!swapped && try_gemv_units(s, d, rc)) return true;
        if (d.algo == MNI_ALGO_GEMV) return false;
        const bool w_batch_ok = s.w_bcount <= 1 || (s.w_bs % 4) == 0;
        bool w_cols = s.w_cs == 1 && (s.w_rs % 4) == 0 && (s.cols % 4) == 0 && aligned16(s.W) && w_batch_ok;
        // (Many small products of 9 to 16 rows: the 16-row form gives a workgroup 256 columns, and under that many most
        // of it idles -- 8192 x (16 x 64 x 16) 109 us against 47 through tiles.  Nor with a short K: 2048 x (16 x 256 x 32)
        // 40 against 43, but 48 against 24 through the outer-product kernel when A is given as its transpose.)
        // (A single narrow product likewise: 16 x 16 x 16384 61 us against 17 through tiles in K slices, 10 x 128 x 16384 59 / 29.)
        // (128 columns and more of a K up to 2048 stay: 9 x 128 x 1024 9.7 against 11.2.)
        if (d.algo == MNI_ALGO_AUTO && s.rows > 8 &&
            (s.cols < 128 || (s.cols < 256 && (s.K > 2048 || s.batch > 1)) || (s.batch > 1 && s.K < 64))) w_cols = false;
        const bool x_batch_ok = s.x_bcount <= 1 || (s.x_bs % 4) == 0;
        // (the pitch of X only matters from the second row on)
        const bool x_dots = s.x_cs == 1 && (s.rows == 1 || (s.x_rs % 4) == 0) && aligned16(s.X) && x_batch_ok;
        const bool w_dots_w = s.w_rs == 1 && (s.w_cs % 4) == 0 && (s.K % 4) == 0 && aligned16(s.W) && w_batch_ok;
        bool w_dots = w_dots_w && x_dots;
        // By itself the dots kernel takes up to 8 rows of a K of at least 512 (see below).  Then it also pays to
        // bring a small operand that is not laid out along K -- the [K, n] weight of a head with a few outputs
        // under a tall activation matrix -- into that layout first, with one small copy launch, when the big
        // operand is worth it (65536 x 768 against [768, 2]: 72 us through the tile kernel, 31 + 3 this way).
        void *packed = nullptr;
        // (At 8 rows the copy eats what the kernel gains over the tile kernel -- unless that kernel is on its slow
        // loads because the row count is not a multiple of 4.)
        if (w_dots_w && !x_dots && !w_cols && d.algo == MNI_ALGO_AUTO && d.split_k <= 1 && (s.rows <= 4 || (s.rows <= 8 && s.rows % 4 != 0)) &&
            s.K >= 512 &&
            (int64_t)s.cols * s.K * s.batch >= (2LL << 20)) {
            const int64_t xb = s.x_bcount > 1 ? s.x_bcount : 1;
            *rc = gemm_ws_alloc(&packed, (size_t)(xb * s.rows * s.K) * sizeof(float));
            if (*rc != MNI_OK) return true;
            const int64_t shape[3] = {xb, s.rows, s.K}, strides[3] = {s.x_bs, s.x_rs, s.x_cs};
            *rc = k_strided_copy((float *)packed, s.X, shape, strides, 3);
            if (*rc != MNI_OK) { gemm_ws_free(packed); return true; }
            s.X = (const float *)packed; s.x_cs = 1; s.x_rs = s.K; s.x_bs = (int64_t)s.rows * s.K;
            w_dots = true;
        }

        if (w_cols) {
            // Slice K until about 4 workgroups per CU exist (every CU streams,
            // nearly all of W is requested at once); a slice is a whole number
            // of workgroup passes.
            const int groups = (s.cols + skinny_cols_block_cols() - 1) / skinny_cols_block_cols();
            s.groups = groups;
            const int pass = skinny_cols_rows_per_pass();
            int split = d.split_k;
            if (split == 0) {
                const int64_t cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
                const int64_t target = 4LL * cus;
                const int64_t have = (int64_t)groups * s.batch;
                split = (int)((target + have - 1) / have);
                const int max_split = (s.K + pass - 1) / pass;
                if (split > max_split) split = max_split;
                if (split < 1) split = 1;
                // Among the counts up to that one, the one whose fullest CU has the fewest rows of K to stream (workgroups on it x
                // rows of a slice, slices being whole passes), and of equals the largest: a K that is not a power of two otherwise
                // leaves the last of the four workgroups of a CU to half of them (1 x 4096 x 14336: 56 slices of 256 rows, 3.5
                // workgroups per CU, 46.8 us; 32 slices of 448, two per CU, 37.6 = 0.78 of HBM).
                if (have <= target) {
                    int best = split;
                    int64_t best_cost = -1;
                    for (int cand = split; cand >= 1; --cand) {
                        int64_t kc = (s.K + cand - 1) / cand;
                        kc = (kc + pass - 1) / pass * pass;
                        const int64_t real = (s.K + kc - 1) / kc;
                        // (never under two workgroups per CU: one, of four wavefronts, keeps too few bytes in flight --
                        // 1 x 5120 x 5120 in 12 slices, 240 workgroups, 25.5 us against 19.7 in 40)
                        if (have * real < 2 * cus && cand != split) continue;
                        const int64_t cost = ((have * real + cus - 1) / cus) * kc;
                        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = cand; }
                    }
                    split = best;
                }
            }
            int kps = (s.K + split - 1) / split;
            kps = (kps + pass - 1) / pass * pass;
            split = (s.K + kps - 1) / kps;
            s.split_k = split; s.k_per_slice = kps;
            // One launch when the partials of a unit can stay inside one XCD's
            // L2 and its arrival flags fit the library's flag array.  Its partial
            // rows are whole 128-byte lines, so that no line is shared by two units.
            DeviceCtx &c = ctx();
            const int64_t flag_count = (int64_t)groups * s.batch * split;
            bool fused = split > 1 && d.algo != MNI_ALGO_SKINNY_TWO_PASS && c.xcd_count > 0 && c.skinny_flags &&
                         flag_count <= (int64_t)c.skinny_flag_cap;
            if (fused) {
                // The reducers of a unit (the workgroups of its last min(rows, slices) slices) wait for all of its
                // slices while they hold their places on the CUs: every reducer of an XCD must fit on it at once,
                // or the first ones could fill it and wait for slices that are never dispatched.
                // With more rows than that leaves room for, a unit gets fewer reducers, each taking several rows.
                const int cus = c.compute_units > 0 ? c.compute_units : 256;
                const int64_t units_per_xcd = ((int64_t)groups * s.batch + c.xcd_count - 1) / c.xcd_count;
                const int64_t room_per_xcd = (int64_t)skinny_cols_fused_occupancy(s) * (cus / c.xcd_count);
                // (Up to 8 rows: 8 x 50304 x 768 33.6 us with 5 reducers per unit against 43.2 in two launches.  Not the
                // 16-row form, one workgroup per CU: 12 x 8192 x 8192 72.5 us with 8 reducers per unit, 58.2 in two launches.)
                const int64_t per_unit = room_per_xcd / units_per_xcd;
                const int64_t wanted = s.rows < split ? s.rows : split;
                fused = s.rows <= 8 ? per_unit >= 1 : per_unit >= wanted;
                s.max_reducers = (int)(per_unit < 16 ? per_unit : 16);
            }
            void *ws = nullptr;
            if (split > 1) {
                const size_t bytes = (size_t)split * s.batch * s.rows * skinny_ws_pitch(s.cols, fused) * sizeof(float);
                *rc = gemm_ws_alloc(&ws, bytes);
                if (*rc != MNI_OK) return true;
                s.ws = (float *)ws;
            }
            if (fused) {
                *rc = next_epoch(&s.epoch);
                s.flags = c.skinny_flags;
            }
            if (*rc == MNI_OK) *rc = launch_skinny_cols(s, fused ? c.xcd_count : 0);
            if (*rc == MNI_OK && split > 1 && !fused) {
                ReduceLaunch r;
                r.ws = s.ws; r.out = s.out; r.bias = s.bias;
                r.slices = split; r.batch = s.batch; r.rows = s.rows; r.cols = s.cols;
                r.o_rs = s.o_rs; r.o_cs = s.o_cs; r.o_bs = s.o_bs;
                r.epilogue = s.epilogue; r.accumulate = s.accumulate; r.bias_on_rows = s.bias_on_rows;
                *rc = launch_skinny_reduce(r);
            }
            gemm_ws_free(ws);
            return true;
        }
        // W contiguous along K: one wavefront per output column.  By itself only up to 8 rows -- its 16-row
        // instantiation is behind the tile kernel's 64 x 64 tiles in K slices on every shape measured (MI355X, us,
        // dots at 9 / 16 rows against tiles: [50304, 768] 80 / 95 against 48, [4096, 4096] 26 / 28 against 24,
        // [1024, 4096] 22 / 25 against 12, [11008, 4096] 56 / 61 against 58).
        // Nor for a short K, where half its lanes have nothing to load (100000 x 128 against 8 columns: 55 us, tiles 22).
        // (One row: from K = 384, 64 x (1 x 4096 x 384) 72 us against 105 through tiles; at K = 256 130 against 144, and the
        // thread-per-output kernel's 121 is ahead of both.)
        if (w_dots && d.split_k <= 1 && ((s.rows <= 8 && (s.K >= 512 || (s.rows == 1 && s.K >= 384))) || d.algo != MNI_ALGO_AUTO)) {
            *rc = launch_skinny_dots(s);
            gemm_ws_free(packed);
            return true;
        }
        gemm_ws_free(packed);
        // Both extents small: the other orientation may be eligible.
        if (attempt == 0 && !swapped && d.N <= 16) swapped = true;
        else break;
    }
    return false;
}

// ---- MFMA path ----------------------------------------------------------------
// Which products go to the register-direct kernel by themselves: 0 = none,
// else the number of wavefronts that share K.
static int direct_plan(const GemmLaunch &g, int cus) {
    // None any more.  The kernel was built for batched products of about one
    // 64 x 64 tile per CU (the backward products of an attention layer), where
    // the tile kernel then spent its time waiting on loads.  Since the tile
    // kernel's K loop carries no vector-ALU work, its 64 x 64 tiles in one K
    // slice are ahead on every such shape (MI355X, microseconds, direct with
    // four wavefronts sharing K against tile): [32 x 512 x 512] x [512 x 64] 16.4
    // vs 13.7, its transposed twin 15.7 vs 13.7, K = 256: 11.5 vs 9.1, K = 1024:
    // 27.4 vs 21.3, 32 x (128 x 128 x 512) 15.4 vs 13.0, 16 x (1024 x 64 x 1024)
    // 27.2 vs 21.5, 40 batches of the first 29.6 vs 20.5.
    // What is left to it: many batches of a few rows and a K of one MFMA phase,
    // where three quarters or more of each 64 x 64 tile of the tile kernel are
    // padding and its LDS round trip is all it does (us, direct with one wavefront
    // against tile): 8192 x (16 x 64 x 16) 32.3 vs 47.5, 2048 x (16 x 256 x 16) 32.0 vs
    // 46.8, 2048 x (32 x 64 x 16) 9.1 vs 15.4, 2048 x (48 x 256 x 16) 39.0 vs 53.2,
    // 512 x (16 x 256 x 16) 8.3 vs 14.2; at K = 32 the two are level.
    // MNI_ALGO_DIRECT selects it for every eligible product.
    if (g.K <= 16 && g.M <= 48 && g.N >= 64 && (int64_t)g.batch * ((g.N + 63) / 64) >= 2 * (int64_t)cus) return 1;
    return 0;
}

// Whether a short-K product of two K-contiguous operands goes to the panel kernel by itself.
static bool panel_plan(const GemmLaunch &g, int cus) {
    // When its 128 x 128 tiles give more than half the CUs a workgroup.  Measured on MI355X against the
    // tile kernel's plans, microseconds: 32 x (512 x 512 x 64) 13.8 vs 19.5, 8 x (1024 x 1024 x 64) 13.0 vs
    // 18.5, 4096 x 4096 x 64 22.3 vs 34.9, K = 32: 9.9 vs 13.7, 16 x (384 x 384 x 64) 8.1 vs 8.7; at
    // 8 x (512 x 512 x 64), 128 tiles, the tile kernel's 64 x 64 tiles are ahead, 7.4 vs 8.0.
    // Not up to 64 rows or columns, where half or more of every tile would be padding (us, panel against 64 x 64 tiles):
    // 64 x (64 x 4096 x 64) 53 / 34, 64 x (4096 x 32 x 64) 49 / 33, 1024 x (64 x 256 x 64) 55 / 37, 256 x (2 x 4096 x 64) 163 / 104;
    // from 96 on it is ahead: 64 x (96 x 4096 x 64) 53 / 62, 1024 x (96 x 96 x 32) 14 / 26, 1024 x (128 x 128 x 64) 29 / 36.
    if (g.M <= 64 || g.N <= 64) return false;
    const int64_t tiles = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * g.batch;
    return tiles * 2 > cus;
}

static void fill_launch(GemmLaunch &g, const mni_gemm_desc &d) {
    g.A = d.A.ptr; g.B = d.B.ptr; g.C = d.C; g.bias = d.bias; g.ws = nullptr;
    g.M = (int)d.M; g.N = (int)d.N; g.K = (int)d.K; g.batch = (int)d.batch;
    g.a_rs = d.A.row_stride; g.a_cs = d.A.col_stride; g.a_bs = d.A.batch_stride;
    g.b_rs = d.B.row_stride; g.b_cs = d.B.col_stride; g.b_bs = d.B.batch_stride;
    g.a_bcount = (int)d.A.batch_count; g.b_bcount = (int)d.B.batch_count;
    g.ldc = d.ldc; g.c_bs = d.c_batch_stride;
    g.epilogue = d.epilogue; g.accumulate = d.accumulate;
}

// What run_mfma would launch for a product, for a caller that wants to know before anything is launched.
struct PlanProbe {
    enum { TILE = 0, PANEL = 1, DIRECT = 2, TILE_FUSED_GELU = 3, TILE_STREAMK = 4, FEWROWS = 5, OUTER = 6 };
    int kind, bm, bn, split, amode, bmode;
    GemmLaunch g;  // kinds TILE and TILE_FUSED_GELU: the launch descriptor, complete
};

// K slices of the few-rows kernel: one workgroup per CU (more gain nothing: with one, the loop already runs close
// to both the memory system's and the matrix pipe's rate), slices of at least 128 K values (four blocks per
// wavefront), at most 32 of them (the last workgroup of a column group adds them up).  Measured against every
// other count on 19 (N, K) pairs from 512 x 512 to 50304 x 768: within 10 % of the best everywhere.
static int fewrows_split(const GemmLaunch &g, int cus) {
    const int64_t groups = (int64_t)((g.N + 127) / 128) * g.batch;
    int64_t split = cus / groups;
    if (split > g.K / 128) split = g.K / 128;
    if (split > 32) split = 32;
    return split < 1 ? 1 : (int)split;
}
// Whether the short-K outer-product kernel is the plan for an eligible product.  It costs what writing C costs
// plus the MFMAs of a wavefront's K pairs, which nothing hides when all wavefronts start together; the tile
// kernel's 64 x 64 tiles pay a fixed prologue and epilogue per tile and little per K step.  Measured on MI355X,
// us, outer against tiles, K = 8 / 32 / 64 / 128: 4096 x 4096 15.3 / 18.1 / 23.8 / 38.0 against 29.0 / 25.9 / 33.0 /
// 46.4; 4096 x 11008 32.6 / 41.0 / 62.2 / 102 against 68.4 / 61.9 / 82.4 / 119; 2048 x 2048 5.7 / 6.9 / 8.9 / 12.3
// against 10.2 / 9.2 / 11.0 / 14.2; 768 x 3072 3.9 / 5.9 / 7.8 / 11.7 against 8.1 / 7.9 / 9.3 / 11.8; 768 x 768
// 3.6 / 5.1 / 7.0 / 10.8 against 5.9 / 5.7 / 6.1 / 7.2.
static bool outer_plan(const GemmLaunch &g, int cus) {
    (void)cus;
    const int64_t outputs = (int64_t)g.M * g.N * g.batch;
    // (K = 192 / 256 / 512: 4096 x 4096 53.9 / 70.4 / 129 against 60.3 / 74.5 / 131, 8192 x 8192 202 / 260 / 497 against 230 /
    // 286 / 510, 2048 x 2048 16.3 / 20.2 / 47.8 against 17.7 / 21.2 / 35.7, 4096 x 11008 156 / 200 / 376 against 156 / 193 / 344)
    // A wavefront's block is 32 x 128, the tile kernel's smallest tile 64 x 64: not where this kernel would pad small
    // or narrow products more than tiles do (us, this kernel against tiles: 2048 x (64 x 64 x 64) 38 / 23,
    // 2048 x (64 x 32 x 64) 39 / 21, 512 x (128 x 64 x 128) 19 / 15; level padding or less: 4096 x (32 x 64 x 32) 24 / 27,
    // 1024 x (80 x 80 x 80) 24 / 45, 2048 x (16 x 256 x 32) 24 / 42, 8192 x (16 x 64 x 16) 28 / 47).
    const int64_t mn = (int64_t)g.M * g.N;
    const int64_t own_pad = (int64_t)((g.M + 31) / 32 * 32) * ((g.N + 127) / 128 * 128);
    const int64_t tile_pad = (int64_t)((g.M + 63) / 64 * 64) * ((g.N + 63) / 64 * 64);
    if (own_pad > tile_pad && own_pad * 9 > mn * 10) return false;
    // (768 x 3072, K = 256: 19.1 against 17.2, so the longest K only from 2048 x 2048 outputs on)
    if (outputs >= (1LL << 22)) return g.K <= 256;
    if (outputs >= (1LL << 21)) return g.K <= 128;
    return outputs >= (1LL << 16) && g.K <= 48;  // (512 x 512: K = 48 5.9 against 6.8, K = 64 6.9 against 6.0)
}
// Whether the few-rows kernel is the plan for an eligible product: from about 512 x 512 of W on it is ahead of the
// tile kernel's 64 x 64 tiles in K slices (us, 32 rows: 512 x 512 7.8 / 15.1, 1024 x 1024 8.8 / 11.7, 4096 x 4096
// 19.1 / 24.4, 8192 x 8192 46.6 / 70.4, 50304 x 768 35.0 / 50.4, 1024 x 16384 24.3 / 29.7); below, and for short K, not.
static bool fewrows_plan(const GemmLaunch &g, int cus) {
    (void)cus;
    return g.K >= 256 && (int64_t)g.N * g.K >= (1 << 18);
}

// Whether the few-rows kernel for a K-contiguous B is the plan for an eligible product.  Measured on MI355X (us, cold W,
// this kernel against the planner's choice without it -- the dots kernel up to 8 rows, 64 x 64 tiles in K slices beyond):
// 16 x 50304 x 768 33.3 / 49.9, 9 rows 32.3 / 49.4, 8 rows 31.9 / 44.8, 4 rows 31.0 / 31.5, 2 rows 29.9 / 29.1, 1 row 31.2 / 28.7;
// 16 x 16384 x 768 13.8 / 16.6, 16 x 8192 x 768 9.5 / 13.1, 16 x 4096 x 768 7.5 / 9.7, 16 x 4096 x 1984 15.5 / 22.7,
// 8 x 32768 x 1984 53.0 / 66.1, 16 x 128256 x 512 70.2 / 74.4, 16 x 32000 x 1024 37.4 / 38.4; behind with a short K, where
// the sum over a wavefront's sixteen blocks at the end of every group of four columns weighs (16 x 65536 x 256 37.3 / 20.2,
// 12 x 262144 x 64 129 / 30), under 4096 columns (12 x 2048 x 1024 10.0 / 9.1), with four rows or fewer
// (4 x 32000 x 1024 36.2 / 29.1) and beyond 16 rows, where eight LDS reads and 32 MFMAs per load add up
// (32 x 50304 x 768 56.4 / 51.3).
// Since A's values for a step are asked of LDS a step ahead (this kernel / the dots kernel up to 8 rows / tiles, us, cold):
// 1 x 50304 x 768 24.9 / 28.8 / 47.8, 4 rows 27.0 / 31.3, 16 rows 33.5, 32 rows 47.2 / - / 53.5; 1 x 16384 x 768 9.9 / 12.1, 4 x 4096 x 768
// 5.3 / 6.9, 4 x 32768 x 1984 42.0 / 50.4, 4 x 2048 x 1024 5.6 / 7.2, 3 x 1024 x 1024 4.7 / 6.3, 2 x 8192 x 640 6.4 / 7.7, 8 x 2048 x 1024 6.4 / 10.2,
// 16 x 2048 x 1024 9.1 / 16.5 / 14.3, 16 x 3072 x 1536 10.6 / 18.4 / 15.6, 20 x 12288 x 768 15.6 / - / 24.1, 32 x 8192 x 768 12.8 / - / 16.8; level at
// 1 x 32000 x 1024 (27.8 / 27.3) and 2 x 4096 x 1984 (9.2 / 9.1); behind at K = 512 and below (4 x 128256 x 512 57.0 / 51.3, 1 x 65536 x 256
// 25.7 / 20.2) and, beyond 16 rows, wherever K is not 768: the steps past the last in the ring of 12 loads multiply zeros, 32 MFMAs each
// (24 x 8192 x 960 17.4 against 15.5, 32 x 32000 x 960 50.4 against 36.5).
// (K beyond 1984: where A still fits LDS -- 2048 values of up to 16 rows, 4096 of up to 8, 8192 of up to 4 -- fewrows_nt_sliced_plan
// decides between this form and the sliced one, and comes first.)
static bool fewrows_nt_plan(const GemmLaunch &g, int cus) {
    (void)cus;
    if (g.M > 16) return g.K == 768 && g.N >= 8192;
    if (g.M > 8) return g.K >= 512 && g.N >= 2048;
    if (g.M > 4) return g.K >= 512 && g.N >= 1024;  // (8 x 1024 x 4096 11.7 against 16.8; 16 rows 21.6 against 12.3)
    return g.K >= 640 && g.N >= 1024;
}
// K slices for the sliced form of that kernel (0: not this form).  A slice is a run of steps of 64 values of K, at most
// as many as the kernel keeps in flight; a workgroup is 64 columns x one slice and has a CU to itself, so a plan costs
// rounds of workgroups x steps of the longest slice, plus something per slice for the sum at the end.
static int fewrows_nt_slices(const GemmLaunch &g, int cus, int want) {
    const int ksteps = g.K / 64, maxs = fewrows_nt_max_steps(g.M);
    const int smin = std::max(2, (ksteps + maxs - 1) / maxs), smax = std::min(ksteps, FEWROWS_NT_MAX_SLICES);
    if (smin > smax) return 0;
    if (want > 0) return want >= smin && want <= smax ? want : 0;
    const int64_t units8 = 8 * (int64_t)(((g.N + 63) / 64 + 7) / 8);
    int best = 0;
    double best_cost = 0.0;
    for (int s = smin; s <= smax; ++s) {
        // a round of workgroups costs its steps (0.7 us each: 256 CUs x 64 columns x 64 values) and about 5 us besides
        // (A into LDS ahead of the first request for W; partial sums acknowledged, counted and added behind the last)
        const int64_t rounds = (units8 * s + cus - 1) / cus;
        const double cost = (double)rounds * ((ksteps + s - 1) / s + 7);
        if (best == 0 || cost < best_cost - 1e-9) { best = s; best_cost = cost; }
    }
    return best;
}
// Measured cold on MI355X (us; the sliced form / the dots kernel / 64 x 64 tiles in K slices), W [N, K]:
//    rows    4096 x 4096        8192 x 8192         32000 x 4096          4096 x 11008        1024 x 8192         4096 x 2048         2048 x 2048
//      1   14.2 / 17.7 / 24.7   49.5 / 54.0 / 87.2   94.9 /  96.5 / 127   36.3 / 43.5 / 64.7   14.3 / 21.4 / 18.2   12.1 / 10.2 / 15.2   12.7 /  8.0 / 14.3
//      4   14.5 / 18.7 / 25.1   51.1 / 55.3 / 88.3   96.7 /  97.6 / 129   38.1 / 44.5 / 65.0   15.1 / 22.9 / 18.4   12.4 / 11.3 / 15.1   13.2 /  9.2 / 14.6
//      8   15.1 / 22.8 / 25.3   53.8 / 61.6 / 88.5  100.3 / 113.7 / 129   41.9 / 51.8 / 65.5   17.1 / 30.6 / 18.9   13.1 / 14.9 / 15.6   14.3 / 12.7 / 14.8
//     16   17.1 / 31.7 / 25.7   62.7 / 88.6 / 89.6  112.5 / 167.5 / 131   52.4 / 67.4 / 66.4   21.9 / 45.2 / 19.1   15.4 / 22.0 / 15.9   17.2 / 20.1 / 15.1
// (the same weights stored [K, N] take 12.2-14.1 us at 4096 x 4096 through the decode product).  With 17 to 32 rows the 32
// MFMAs per load weigh: 41-45 us against the tiles' 28 at 4096 x 4096.  Where LDS holds all of A's K the unsliced form is the third
// choice, and from about 5000 columns on the first: 1 x 32000 x 4096 81.9, 1 x 8192 x 8192 45.5, 8 x 32000 x 4096 84.8, 8 x 14336 x 4096 41.6,
// 1 x 2048 x 2048 6.5, 4 x 4096 x 2048 9.5, 8 x 4096 x 2048 10.4, 16 x 4096 x 2048 14.0.
static bool fewrows_nt_sliced_plan(const GemmLaunch &g, int cus) {
    (void)cus;
    // (up to there the unsliced form holds A in LDS: 2048 values of up to 16 rows, 4096 of up to 8, 8192 of up to 4)
    const int kmax = FEWROWS_NT_LDS_FLOATS / (g.M > 8 ? 16 : g.M > 4 ? 8 : 4) - 16;
    if (g.M > 16 || (int64_t)g.N * g.K < (1 << 23)) return false;
    // Where the unsliced form holds A it is ahead from about 5000 columns on -- nothing to add up, no rounds of workgroups (us,
    // unsliced / sliced: 8 x 5120 x 4096 19.7 / 25.1, 4 x 6144 x 4096 20.8 / 24.3, 4 x 8192 x 8192 47.2 / 51.1, 8 x 14336 x 4096 41.7 / 51.0,
    // 1 x 32000 x 4096 81.9 / 94.7, 16 x 16384 x 2048 29.9 / 32.0) -- and behind at 4096, where three wavefronts in four have no group
    // of columns (4 x 4096 x 4096 16.0 / 14.5, 8 rows 17.4 / 15.1).
    if (g.K <= kmax && (g.N >= 5120 || g.K <= 2048)) return false;
    return g.M > 8 ? g.N >= 2048 : (g.K >= 4096 || g.M >= 8);
}
// Whether run_mfma gives the product to the sliced form by itself.
static bool fewrows_nt_sliced_takes(const GemmLaunch &g, int amode, int bmode) {
    DeviceCtx &c = ctx();
    const int cus = c.compute_units > 0 ? c.compute_units : 256;
    if (!gemm_fewrows_nt_sliced_eligible(g, amode, bmode) || c.xcd_count != 8 || (size_t)((g.N + 63) / 64 + 7) > c.fewrows_counter_cap) return false;
    if (!fewrows_nt_sliced_plan(g, cus)) return false;
    const int fs = fewrows_nt_slices(g, cus, 0);
    // (a caller that cannot allocate gets the plan only when the fixed scratch holds its partial sums)
    return fs > 0 && !(c.scratch && fewrows_nt_sliced_ws_floats(g.N, fs) * sizeof(float) > c.scratch_bytes);
}
// Whether run_mfma would give the product to the few-rows kernel by itself.
static bool fewrows_takes(const mni_gemm_desc &d) {
    if (d.K == 0 || d.epilogue >= MNI_EPI_BIAS_GELU_DUAL) return false;
    GemmLaunch g;
    fill_launch(g, d);
    DeviceCtx &c = ctx();
    const int amode = classify(g.a_cs, g.a_rs), bmode = classify(g.b_rs, g.b_cs);
    const int cus = c.compute_units > 0 ? c.compute_units : 256;
    if (gemm_fewrows_nt_eligible(g, amode, bmode) && fewrows_nt_plan(g, cus)) return true;  // (its twin for a K-contiguous B)
    if (fewrows_nt_sliced_takes(g, amode, bmode)) return true;
    return gemm_fewrows_eligible(g, amode, bmode) && (size_t)((g.N + 127) / 128) * g.batch <= c.fewrows_counter_cap && c.xcd_count == 8 &&
           fewrows_plan(g, cus);
}

// K slices for a product of `tiles` 64 x 64 tiles (at most one per CU) of `ktiles` K steps each.
// Estimated microseconds of a plan with s slices:
//   (per_cu (steps + 3) + 3) c  +  [s > 1]  (2.5 + 2 s out_bytes / 5 TB/s)
// per_cu = workgroups on the fullest CU, steps = K steps per slice, c = 0.55 us per K step of a workgroup that
// has its CU to itself and 0.48 when several share one (they cover each other's barriers and LDS round trips);
// three steps' worth of prologue and epilogue per workgroup and per launch; the reduction pass costs a launch
// and reads what the slices wrote.  Fitted to, and within 10 % of, 60 measured plans: M = 24..384 against
// (N, K) = (4096, 4096), (4096, 1024), (1024, 4096), (11008, 4096), (4096, 11008), s = 1..16; e.g.
// 64 x 4096 x 4096: s = 1, 2, 4, 8, 16 measured 68.0 / 40.2 / 25.4 / 26.7 / 30.5 us, estimated 73.7 / 41.8 / 25.1 /
// 25.6 / 31.8.  The smallest s within 3 % of the best estimate wins; slices keep at least 8 K steps (2 when K has at most 32).
static int split_for_few_tiles(int64_t tiles, int ktiles, int cus, int64_t out_bytes) {
    static const int cand[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64};
    double best = 0.0;
    int best_s = 1;
    for (int s : cand) {
        // (Up to 32 K steps a slice may be as short as two: 64 x 512 x 512 in 1 / 2 / 4 / 8 slices measured 12.9 / 11.1 / 8.7 /
        // 8.4 us, estimated 12.1 / 10.2 / 8.0 / 6.9; 256 x 512 x 512 13.0 / 11.4 / 9.3 / 9.6; 64 x 1024 x 256 8.9 / 9.2 / 7.9 / 8.4.)
        if (s > 1 && ktiles / s < (ktiles <= 32 ? 2 : 8)) break;
        const int64_t per_cu = (tiles * s + cus - 1) / cus;
        const int steps = (ktiles + s - 1) / s;
        double t = ((double)per_cu * (steps + 3) + 3) * (per_cu > 1 ? 0.48 : 0.55);
        if (s > 1) t += 2.5 + 2.0 * s * (double)out_bytes / 5.0e6;
        if (s == 1 || t < best * 0.97) {
            best = t;
            best_s = s;
        }
    }
    return best_s;
}

static int run_mfma(const mni_gemm_desc &d, PlanProbe *probe = nullptr) {
    GemmLaunch g;
    fill_launch(g, d);
    const int bk = gemm_mfma_tile_k();
    DeviceCtx &c = ctx();
    const int cus = c.compute_units > 0 ? c.compute_units : 256;
    const int ktiles = (g.K + bk - 1) / bk;
    const bool sk_device = c.xcd_count > 0 && c.skinny_flags && cus % c.xcd_count == 0;

    // op(A)(m, k): K stride = col_stride, M stride = row_stride.
    const int amode = g.K == 0 ? 2 : classify(g.a_cs, g.a_rs);
    // op(B)(k, n): K stride = row_stride, N stride = col_stride.
    const int bmode = g.K == 0 ? 2 : classify(g.b_rs, g.b_cs);

    // Short-K panel form: forced, or chosen when its 128 x 128 tiles fill the machine.
    if (d.algo == MNI_ALGO_PANEL || (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && d.epilogue < MNI_EPI_BIAS_GELU_DUAL &&
                                     gemm_panel_eligible(g, amode, bmode) && panel_plan(g, cus))) {
        if (!gemm_panel_eligible(g, amode, bmode))
            return set_error(MNI_ERR_INVALID, "sgemm: the short-K panel kernel takes two K-contiguous operands with K <= 64, K %% 4 == 0");
        if (d.split_k > 1) return set_error(MNI_ERR_INVALID, "sgemm: the short-K panel kernel takes no split_k");
        g.tiles_m = (g.M + 127) / 128;
        g.tiles_n = (g.N + 127) / 128;
        g.split_k = 1;
        g.k_per_slice = g.K;
        g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_flags = nullptr; g.sk_epoch = 0; g.status = c.status_dev;
        if (probe) { probe->kind = PlanProbe::PANEL; return MNI_OK; }
        return launch_gemm_panel(g, amode, bmode);
    }
    // Short-K outer-product form (both operands contiguous along the output axes): forced, or chosen by outer_plan.
    if (d.algo == MNI_ALGO_OUTER || (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && gemm_outer_eligible(g) && outer_plan(g, cus))) {
        if (!gemm_outer_eligible(g))
            return set_error(MNI_ERR_INVALID, "sgemm: the short-K outer-product kernel takes an A contiguous along M and a B contiguous along N, "
                                              "K <= 512, N %% 4 == 0, B and C 16-byte aligned, no epilogue");
        if (d.split_k > 1) return set_error(MNI_ERR_INVALID, "sgemm: the short-K outer-product kernel takes no split_k");
        g.tiles_m = (g.M + 127) / 128;
        g.tiles_n = (g.N + 127) / 128;
        g.split_k = 1;
        g.k_per_slice = g.K;
        g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_flags = nullptr; g.sk_epoch = 0; g.status = c.status_dev;
        if (probe) { probe->kind = PlanProbe::OUTER; return MNI_OK; }
        return launch_gemm_outer(g);
    }
    // The same in K slices: forced with a split_k or a K beyond the unsliced form's LDS, or chosen by fewrows_nt_sliced_plan.
    {
        const bool fs_ok = gemm_fewrows_nt_sliced_eligible(g, amode, bmode) && c.xcd_count == 8 && (size_t)((g.N + 63) / 64 + 7) <= c.fewrows_counter_cap;
        int fs = 0;
        if (d.algo == MNI_ALGO_FEWROWS_NT && (d.split_k > 1 || !gemm_fewrows_nt_eligible(g, amode, bmode))) {
            fs = fs_ok ? fewrows_nt_slices(g, cus, d.split_k > 1 ? d.split_k : 0) : 0;
            if (fs == 0)
                return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel for a K-contiguous B takes one product of up to 32 rows of a K-contiguous A, operands "
                                                  "16-byte aligned, K %% 64 == 0; at most 8192 / 4096 / 2048 / 960 for up to 4 / 8 / 16 / 32 rows in one piece, or in 2 to 16 slices (split_k) of at "
                                                  "most 1024 (768) each");
        } else if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && fewrows_nt_sliced_takes(g, amode, bmode)) {
            fs = fewrows_nt_slices(g, cus, 0);
        }
        if (fs > 0) {
            if (probe) { probe->kind = PlanProbe::FEWROWS; return MNI_OK; }
            void *fws = nullptr;
            MNI_TRY(gemm_ws_alloc(&fws, fewrows_nt_sliced_ws_floats(g.N, fs) * sizeof(float)));
            const int rc = launch_gemm_fewrows_nt_sliced(g, amode, bmode, fs, (float *)fws, c.fewrows_counters);
            gemm_ws_free(fws);
            return rc;
        }
    }
    // Few rows against a wide K-contiguous operand (a weight stored [out, in]): forced, or chosen by fewrows_nt_plan.
    if (d.algo == MNI_ALGO_FEWROWS_NT || (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && gemm_fewrows_nt_eligible(g, amode, bmode) && fewrows_nt_plan(g, cus))) {
        if (!gemm_fewrows_nt_eligible(g, amode, bmode) || d.split_k > 1)
            return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel for a K-contiguous B takes one product of up to 32 rows of a K-contiguous A, K %% 64 == 0 and "
                                              "short enough for A to sit in LDS (8192 / 4096 / 2048 / 960 for up to 4 / 8 / 16 / 32 rows), operands 16-byte aligned, no split_k");
        if (probe) { probe->kind = PlanProbe::FEWROWS; return MNI_OK; }
        return launch_gemm_fewrows_nt(g, amode, bmode);
    }
    // Few-rows form (9 to 32 rows against a wide N-contiguous operand): forced, or chosen by fewrows_plan.
    {
        // (its K slices meet in one XCD's L2: the workgroup-to-XCD mapping must be the confirmed round-robin over 8)
        const bool fr_ok = gemm_fewrows_eligible(g, amode, bmode) && (size_t)((g.N + 127) / 128) * g.batch <= c.fewrows_counter_cap && c.xcd_count == 8;
        int fr_split = 0;
        if (d.algo == MNI_ALGO_FEWROWS) {
            if (!fr_ok)
                return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel takes 9 to 32 rows of a K-contiguous A against an N-contiguous B, "
                                                  "K %% 8 == 0, N %% 4 == 0, 16-byte aligned");
            fr_split = d.split_k > 0 ? d.split_k : fewrows_split(g, cus);
        } else if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && fr_ok && fewrows_plan(g, cus)) {
            fr_split = fewrows_split(g, cus);
        }
        if (fr_split > 0) {
            g.tiles_m = 1;
            g.tiles_n = (g.N + 127) / 128;
            const int per = ((g.K + fr_split - 1) / fr_split + 31) / 32 * 32;
            g.k_per_slice = per;
            g.split_k = (g.K + per - 1) / per;
            g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_epoch = 0; g.status = c.status_dev;
            g.sk_flags = c.fewrows_counters;
            if (probe) { probe->kind = PlanProbe::FEWROWS; return MNI_OK; }
            void *fws = nullptr;
            if (g.split_k > 1) {
                MNI_TRY(gemm_ws_alloc(&fws, (size_t)g.split_k * g.batch * g.M * g.N * sizeof(float)));
                g.ws = (float *)fws;
            }
            const int rc = launch_gemm_fewrows(g, amode, bmode);
            gemm_ws_free(fws);
            return rc;
        }
    }
    // Register-direct form: forced, or chosen for batched products of many small tiles.
    {
        int ksplit = 0;
        if (d.algo == MNI_ALGO_DIRECT) {
            if (!gemm_direct_eligible(g, amode, bmode))
                return set_error(MNI_ERR_INVALID, "sgemm: operand layouts not eligible for the direct kernel (each operand "
                                                  "contiguous along K with K %% 4 == 0, or along M / N with an even extent)");
            if (d.split_k != 0 && d.split_k != 1 && d.split_k != 4)
                return set_error(MNI_ERR_INVALID, "sgemm: the direct kernel takes split_k 0, 1 or 4");
            ksplit = d.split_k == 4 ? 4 : 1;
        } else if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && d.epilogue < MNI_EPI_BIAS_GELU_DUAL && gemm_direct_eligible(g, amode, bmode)) {
            ksplit = direct_plan(g, cus);
        }
        if (ksplit) {
            g.tiles_m = (g.M + 63) / 64;
            g.tiles_n = (g.N + 63) / 64;
            g.split_k = 1;
            g.k_per_slice = g.K;
            g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_flags = nullptr; g.sk_epoch = 0; g.status = c.status_dev;
            if (probe) { probe->kind = PlanProbe::DIRECT; return MNI_OK; }
            return launch_gemm_direct(g, amode, bmode, ksplit);
        }
    }

    // Can the K steps of tiles of this shape be dealt over the stream-K grid?
    // In every XCD's stream-K region each workgroup must own at least
    // `min_steps` K steps (with none, a finisher would wait for a partial that
    // nobody writes; with few, the fix-up costs more than it saves).
    auto streamk_fits = [&](int tm, int tn, int min_steps) {
        if (!sk_device || ktiles <= 0 || d.split_k > 1) return false;
        const int64_t wpx = (int64_t)cus / c.xcd_count * gemm_mfma_resident_per_cu(tm, tn);
        const int64_t total = (int64_t)((g.M + tm - 1) / tm) * ((g.N + tn - 1) / tn) * g.batch;
        if (total * ktiles > 0x7fffffffLL || wpx > 256 || (size_t)(wpx * c.xcd_count) > c.skinny_flag_cap) return false;
        for (int64_t xt = total / c.xcd_count; xt <= (total + c.xcd_count - 1) / c.xcd_count; ++xt) {
            const int64_t left = xt % wpx;
            const int64_t region = left == 0 ? 0 : (xt >= wpx ? left + wpx : left);
            if (region > 0 && region * ktiles < wpx * min_steps) return false;
        }
        return true;
    };

    // Tile shape and work distribution.  A side is 64 wide when that extent is
    // at most 64 (no half-empty tiles).  Otherwise: one workgroup per tile of
    // the biggest shape that deals the CUs equal loads; failing that, stream-K
    // (which has no rounds to fill) over 128 x 128 tiles when there are more of
    // them than workgroup slots and over 64 x 64 tiles when not; else (device
    // mapping unknown, tiny product) K slices and a reduction pass.
    int bm = g.M <= 64 ? 64 : 128, bn = g.N <= 64 ? 64 : 128;
    bool streamk = false;
    bool whole_tiles = false;  // one workgroup per tile, no K slices
    int planned_split = 0;     // K slices chosen by the planner (0: by the slot rule further down)
    // The two-output and the gelu'-scaling epilogues exist in the one-workgroup-per-tile form only;
    // strip sums for the bias gradient are laid out for 128-row tiles.
    const bool fused_gelu = d.epilogue >= MNI_EPI_BIAS_GELU_DUAL;
    if (fused_gelu) {
        whole_tiles = true;
        if (d.algo == MNI_ALGO_MFMA_SMALL) bm = bn = 64;
        if (d.colsum_part) bm = 128;
    } else if (d.algo == MNI_ALGO_MFMA_SMALL) {
        bm = bn = 64;
    } else if (d.algo == MNI_ALGO_AUTO || d.algo == MNI_ALGO_MFMA_STREAMK) {
        const int64_t big_tiles = (int64_t)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * g.batch;
        const int64_t big_slots = (int64_t)cus * gemm_mfma_resident_per_cu(bm, bn);
        // One workgroup per tile when some tile shape deals the CUs equal loads: a CU's matrix pipe is
        // shared by the workgroups resident on it, so what counts is tiles per CU, not per workgroup slot
        // (768 tiles of 128 x 128 on 256 CUs run as fast per tile as 1024 do).  The biggest shape whose last
        // round is at least 95 % full wins; at least two tiles per CU, except that 128 x 128 tiles may come one
        // per CU when K is 1024 and more.  (Measured: whole tiles take ideal / fill, stream-K ideal x 1.03-1.05;
        // 2560^3 with 64 x 64 tiles at 89 % loses 10 % to stream-K, 4096 x 768 x 3072 with 64 x 64 tiles at 100 % beats
        // it by 10 %.)  Big before small whatever the K: on operands of normally distributed values, us, 128 x 128
        // against what smaller tiles the same rule picked before: 4096 x 4096 x 1024 247.9 / 262.2 (64 x 64), x 512
        // 133.4 / 140.9, 4096 x 3072 x 768 146.0 / 151.2, 4096 x 1024 x 4096 239.7 / 248.7 (128 x 64, two per CU), its
        // transposed forms 238-243 / 248-251.  An earlier version of this rule preferred the small shapes up to 32 K
        // steps on the strength of products of constants (4096 x 4096 x 1024: 244.6 / 246.5 there): constants toggle few
        // bits, the matrix pipe draws less and clocks higher, and the ranking of the tile shapes turns round.
        if (ktiles >= 8 && d.split_k == 0 && d.algo == MNI_ALGO_AUTO) {
            const int cand[4][2] = {{128, 128}, {128, 64}, {64, 128}, {64, 64}};
            for (int i = 0; i < 4 && !whole_tiles; ++i) {
                const int cm = cand[i][0], cn = cand[i][1];
                if (cm > bm || cn > bn) continue;
                const int64_t tiles = (int64_t)((g.M + cm - 1) / cm) * ((g.N + cn - 1) / cn) * g.batch;
                const int64_t per_cu = (tiles + cus - 1) / cus;
                const bool alone_ok = cm == 128 && cn == 128 && g.K >= 1024;  // (one 128 x 128 workgroup per CU, a K long enough to hide its start and end)
                if ((per_cu >= 2 || alone_ok) && tiles * 100 >= per_cu * cus * 95) {
                    whole_tiles = true;
                    bm = cm;
                    bn = cn;
                }
            }
        }
        if (whole_tiles) {
            // settled above
        } else if (ktiles >= 8 && d.split_k == 0 && sk_device) {
            const bool long_k = big_tiles * ktiles >= 20 * big_slots;
            if (long_k && big_tiles >= big_slots) {
                // more big tiles than workgroup slots and plenty of K steps per slot: stream-K over big tiles
                streamk = streamk_fits(bm, bn, 8);
            } else if (long_k && ktiles >= 512 && big_tiles * 16 < 3 * big_slots && ((int64_t)g.M + g.N) * g.K * 4 > (128LL << 20)) {
                // A handful of big tiles over a K so long that the operands outgrow the Infinity Cache:
                // 64 x 64 tiles would stream them twice as often (1024 x 1024 x 65536: 1127 us against
                // 1015 us for 128 x 128 tiles in K slices, the plan below)
            } else {
                const int64_t tiles64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64) * g.batch;
                const int64_t wide = g.N % 128 == 0 ? (int64_t)(g.N / 128) : 0;  // 64 x 128 tiles of a product of up to 64 rows
                if (g.M > 32 && g.M <= 64 && g.batch == 1 && tiles64 <= cus && wide > 0 && cus % wide == 0 && cus / wide <= 16 &&
                    ktiles >= 8 * (cus / wide) && (int64_t)g.N * g.K >= (1LL << 24)) {
                    // 33 to 64 rows against a weight that outgrows the L2s (batched decoding; the weight comes from HBM):
                    // 64 x 128 tiles in as many K slices as give every CU one workgroup read B in 512-byte pieces of a row,
                    // which is what streams best.  Cold B, us, against 64 x 64 tiles in the slices of the model below:
                    // 64 x 4096 x 4096 25.6 / 27.4, 33 rows 25.2 / 27.0, 64 x 8192 x 8192 69.8 / 73.1, 64 x 4096 x 8192 40.1 / 45.3,
                    // 64 x 8192 x 2048 25.1 / 27.1, 64 x 2048 x 8192 26.2 / 29.6, 64 x 4096 x 11008 50.5 / 52.1 (with B in the
                    // Infinity Cache the small tiles are 3 % ahead: 23.3 / 24.1 at 4096 x 4096).  Below 2^24 elements of B the
                    // small tiles lead: 64 x 2048 x 4096 17.8 / 17.1, 4096 x 2048 17.2 / 16.4, 8192 x 1024 17.2 / 16.6, 2048 x 2048 15.8 / 12.7.
                    bm = 64;
                    bn = 128;
                    planned_split = (int)(cus / wide);
                    whole_tiles = planned_split == 1;
                } else if (g.M > 64 && g.M <= 128 && g.batch == 1 && tiles64 <= cus && wide > 0 && cus % wide == 0 && cus / wide <= 16 &&
                           ktiles >= 8 * (cus / wide) && g.K >= 8192 && (int64_t)g.N * g.K >= (1LL << 25)) {
                    // 65 to 128 rows against a long K of a large weight: the same with 128 x 128 tiles.  Cold B, us, against
                    // 64 x 64 tiles: 128 x 8192 x 8192 126.8 / 133.8, 80 rows 125.1 / 132.5, 128 x 4096 x 8192 69.4 / 71.4,
                    // 128 x 4096 x 11008 89.2 / 92.8; level at 4096 x 4096 and 2048 x 8192, behind at 8192 x 2048 and shorter K.
                    bm = 128;
                    bn = 128;
                    planned_split = (int)(cus / wide);
                    whole_tiles = planned_split == 1;
                } else if (tiles64 <= cus) {
                    // At most one 64 x 64 tile per CU: K slices by the cost model of split_for_few_tiles (one
                    // slice, i.e. no reduction pass, wins for short K: 32 x (512 x 64 x 512) 13.7 us whole, 19.0 in
                    // two K slices, 19.8 stream-K; several for long K: 128 x 4096 x 4096 69.6 us whole, 40.1 in four).
                    bm = bn = 64;
                    planned_split = split_for_few_tiles(tiles64, ktiles, cus, (int64_t)g.M * g.N * g.batch * 4);
                    whole_tiles = planned_split == 1;
                } else if (tiles64 <= 2LL * cus && ktiles <= 32) {
                    // up to two per CU, of a short K: one workgroup per tile (40 batches of the product above,
                    // 1.25 tiles per CU: 20.6 us whole, 27.5 stream-K)
                    bm = bn = 64;
                    whole_tiles = true;
                } else {
                    streamk = streamk_fits(64, 64, 8);
                    if (streamk) {
                        bm = bn = 64;
                    } else if (ktiles <= 32) {
                        // too few K steps to deal: whole 64 x 64 tiles all the same, the last round part empty
                        // (768 x 3072 x 256, 576 tiles: 17.5 us against 24.4 for 128 x 128 tiles in K slices)
                        bm = bn = 64;
                        whole_tiles = true;
                    }
                }
            }
        } else {
            // short K, a requested split, or no stream-K on this device: 64 x 64 when
            // 128 x 128 tiles would leave the machine with few, short-lived workgroups
            const int64_t t128 = (int64_t)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * g.batch;
            const int64_t big_split = d.split_k > 0 ? d.split_k : (ktiles / 8 > 0 ? ktiles / 8 : 1);
            // (fewer than 8 K steps: 64 x 64 whatever the tile count -- a tile is mostly prologue and epilogue, and the
            // small ones overlap them better; in every layout 4096 x 11008 x 64 98 -> 82 us, 8192 x 8192 x 128 187 -> 173,
            // 2048 x 8192 x 32 30.6 -> 26.8, 4096 x 4096 x 192 62 -> 60)
            if ((bm == 128 || bn == 128) && ((ktiles < 8 && d.split_k == 0) || (g.K <= 256 && t128 < 4LL * cus) || t128 * big_split < 2LL * cus))
                bm = bn = 64;
        }
        if (d.algo == MNI_ALGO_MFMA_STREAMK && !streamk) {
            if (!sk_device) return set_error(MNI_ERR_INVALID, "sgemm: stream-K needs a confirmed workgroup-to-XCD mapping");
            if (d.split_k > 1) return set_error(MNI_ERR_INVALID, "sgemm: stream-K does not take a split_k");
            if (!streamk_fits(bm, bn, 1)) return set_error(MNI_ERR_INVALID, "sgemm: product too small for the stream-K grid");
            streamk = true;
        }
    }
    g.tiles_m = (g.M + bm - 1) / bm;
    g.tiles_n = (g.N + bn - 1) / bn;

    g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_flags = nullptr; g.sk_epoch = 0; g.status = c.status_dev;
    if (fused_gelu) {
        g.split_k = 1;
        g.k_per_slice = g.K > 0 ? g.K : 1;
        g.aux_out = d.aux;                // shares its slot with the K-slice partials, which this form never has
        g.colsum_part = d.colsum_part;    // shares its slot with the stream-K marks
        if (probe) {
            probe->kind = PlanProbe::TILE_FUSED_GELU;
            probe->bm = bm; probe->bn = bn; probe->split = 1; probe->amode = amode; probe->bmode = bmode;
            probe->g = g;
            return MNI_OK;
        }
        return launch_gemm_mfma(g, amode, bmode, bm, bn);
    }
    void *ws = nullptr;
    if (streamk) {
        if (probe) { probe->kind = PlanProbe::TILE_STREAMK; return MNI_OK; }
        g.split_k = 1;
        g.k_per_slice = g.K;
        g.streamk = 1;
        g.sk_xcds = c.xcd_count;
        g.sk_wpx = cus / c.xcd_count * gemm_mfma_resident_per_cu(bm, bn);
        g.sk_flags = c.skinny_flags;
        MNI_TRY(next_epoch(&g.sk_epoch));
        MNI_TRY(gemm_ws_alloc(&ws, (size_t)g.sk_xcds * g.sk_wpx * bm * bn * sizeof(float)));
        g.ws = (float *)ws;
        const int rc = launch_gemm_mfma(g, amode, bmode, bm, bn);
        gemm_ws_free(ws);
        return rc;
    }

    // Split K when the output tiles alone cannot fill the machine (two
    // workgroups fit on each CU).  Slices are whole K steps.
    int split = whole_tiles ? 1 : (planned_split > 0 && d.split_k == 0 ? planned_split : d.split_k);
    if (split == 0) {
        const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n * g.batch;
        const int64_t slots = (bm * bn >= 128 * 128 ? 2LL : 4LL) * cus;
        split = 1;
        if (tiles * 4 < slots * 3) {
            split = (int)((slots + tiles - 1) / tiles);
            const int max_split = ktiles / 8 > 0 ? ktiles / 8 : 1;  // >= 8 K steps per slice
            if (split > max_split) split = max_split;
            if (split > 64) split = 64;
        }
    }
    if (split > ktiles) split = ktiles > 0 ? ktiles : 1;
    int tiles_per_slice = ktiles > 0 ? (ktiles + split - 1) / split : 1;
    split = ktiles > 0 ? (ktiles + tiles_per_slice - 1) / tiles_per_slice : 1;
    g.split_k = split;
    g.k_per_slice = split > 1 ? tiles_per_slice * bk : (g.K > 0 ? g.K : 1);
    if (probe) {
        probe->kind = PlanProbe::TILE;
        probe->bm = bm; probe->bn = bn; probe->split = split; probe->amode = amode; probe->bmode = bmode;
        probe->g = g;
        return MNI_OK;
    }

    if (split > 1) {
        const size_t bytes = (size_t)split * g.batch * g.M * g.N * sizeof(float);
        MNI_TRY(gemm_ws_alloc(&ws, bytes));
        g.ws = (float *)ws;
    }
    int rc = launch_gemm_mfma(g, amode, bmode, bm, bn);
    if (rc == MNI_OK && split > 1)
        rc = finish_split(g.ws, g.C, g.bias, split, g.batch, g.M, g.N, g.ldc, 1, g.c_bs, g.epilogue, g.accumulate, 0);
    gemm_ws_free(ws);
    return rc;
}

int sgemm(const mni_gemm_desc &d) {
    MNI_TRY(ensure_init());
    MNI_TRY(validate(d));
    if (d.M == 0 || d.N == 0 || d.batch == 0) return MNI_OK;
    // Batches of A against one shared B, stacked at a uniform row pitch in A and in C (x[B, T, d] . W[d, n], and the
    // dX of it): one product of B x T rows.  As a batch of small products every batch pads its few rows to a tile
    // and reads B again ([1024, 1, 4096] . [4096, 4096]: 6.5 ms as 1024 products of one row, 0.3 as one of 1024 rows).
    if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && d.batch > 1 && d.B.batch_count == 1 && d.A.batch_count == d.batch &&
        d.A.batch_stride == d.M * d.A.row_stride &&
        d.c_batch_stride == d.M * d.ldc && d.epilogue <= MNI_EPI_BIAS_GELU && d.M * d.batch <= 0x7fffffffLL) {
        mni_gemm_desc one = d;
        one.M = d.M * d.batch;
        one.batch = 1;
        one.A.batch_count = 1;
        return sgemm(one);
    }
    // An operand that is contiguous along M or N is read in 16-byte pieces along that axis, which an edge tile can
    // only do when the edge falls on a multiple of 4; otherwise its workgroups take the element-wise loop, several
    // times slower, and the whole launch waits for them (2048 x 2050 x 2048: 181 us against 134 for 2048 columns).
    // A big product with such an edge is cut into the part that ends on a multiple of 4 and a strip of 1 to 3 columns
    // (rows), which goes down the path of products with a few output columns (rows).
    if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && d.epilogue <= MNI_EPI_BIAS_GELU && d.K > 0 &&
        2.0 * (double)d.M * (double)d.N * (double)d.K * (double)d.batch >= 6e9) {
        if (d.B.col_stride == 1 && d.B.row_stride != 1 && d.N % 4 != 0 && d.N >= 64) {
            const int64_t n0 = d.N - d.N % 4;
            mni_gemm_desc main = d, strip = d;
            main.N = n0;
            strip.N = d.N - n0;
            strip.B.ptr = d.B.ptr + n0;
            strip.C = d.C + n0;
            if (d.bias) strip.bias = d.bias + n0;
            MNI_TRY(sgemm(main));
            return sgemm(strip);
        }
        if (d.A.row_stride == 1 && d.A.col_stride != 1 && d.M % 4 != 0 && d.M >= 64) {
            const int64_t m0 = d.M - d.M % 4;
            mni_gemm_desc main = d, strip = d;
            main.M = m0;
            strip.M = d.M - m0;
            strip.A.ptr = d.A.ptr + m0;
            strip.C = d.C + m0 * d.ldc;
            MNI_TRY(sgemm(main));
            return sgemm(strip);
        }
    }
    if (d.algo == MNI_ALGO_TINY || (d.algo == MNI_ALGO_AUTO && d.split_k == 0)) {
        // A product that a launch's worth of threads computes outright (the README example's sizes: measured
        // 2-3 us each against 4-13 us through the skinny and tile kernels).
        GemmLaunch g;
        fill_launch(g, d);
        g.tiles_m = g.tiles_n = 1; g.split_k = 1; g.k_per_slice = g.K > 0 ? g.K : 1;
        g.streamk = 0; g.sk_wpx = 0; g.sk_xcds = 0; g.sk_flags = nullptr; g.sk_epoch = 0; g.status = ctx().status_dev;
        if (d.algo == MNI_ALGO_TINY) {
            if (d.epilogue > MNI_EPI_BIAS_GELU || d.split_k > 1)
                return set_error(MNI_ERR_INVALID, "sgemm: the tiny-product kernel takes no split_k and no fused GELU epilogue");
            return launch_gemm_tiny(g);
        }
        if (gemm_tiny_eligible(g)) return launch_gemm_tiny(g);
    }
    // 9 to 16 rows against a wide N-contiguous operand: the few-rows MFMA kernel is level with or ahead of the skinny
    // kernel's 16-row forms (us, few-rows against skinny: 16 x 4096 x 4096 18.6 / 21.5, 12 rows 18.6 / 30.5,
    // 16 x 8192 x 8192 46 / 58, 16 x 1024 x 1024 8.5 / 8.4; at 8 rows the skinny kernel leads, 15.2 / 18.6)
    // 9 to 32 rows of the decode shape come first: there the 16 x 16 x 4 form of the decode product is ahead of both
    // (16 x 4096 x 4096 14.1 us, 32 rows 16.5)
    if ((d.algo == MNI_ALGO_AUTO || d.algo == MNI_ALGO_GEMV) && d.split_k == 0 && d.M > 8 && d.M <= 32 && d.batch == 1 && d.K > 0 &&
        d.epilogue <= MNI_EPI_BIAS_GELU) {
        SkinnyLaunch s;
        s.rows = (int)d.M; s.cols = (int)d.N; s.K = (int)d.K; s.batch = 1;
        s.X = d.A.ptr; s.x_rs = d.A.row_stride; s.x_cs = d.A.col_stride; s.x_bs = 0; s.x_bcount = 1;
        s.W = d.B.ptr; s.w_rs = d.B.row_stride; s.w_cs = d.B.col_stride; s.w_bs = 0; s.w_bcount = 1;
        s.out = d.C; s.o_rs = d.ldc; s.o_cs = 1; s.o_bs = 0; s.bias = d.bias; s.bias_on_rows = 0;
        s.epilogue = d.epilogue; s.accumulate = d.accumulate;
        s.ws = nullptr; s.split_k = 1; s.k_per_slice = s.K; s.groups = 0; s.flags = nullptr; s.epoch = 0; s.max_reducers = 16; s.status = ctx().status_dev;
        int rc16 = MNI_OK;
        if (try_gemv_units(s, d, &rc16)) return rc16;
    }
    // (the sliced form of the kernel for a K-contiguous B also takes 1 to 4 rows: 4 x 4096 x 4096 14.6 us against the dots kernel's 18.7)
    const bool to_fewrows = d.algo == MNI_ALGO_AUTO && d.split_k == 0 && d.M <= 32 && fewrows_takes(d);
    if (!to_fewrows &&
        ((d.algo == MNI_ALGO_AUTO && d.epilogue < MNI_EPI_BIAS_GELU_DUAL) || d.algo == MNI_ALGO_SKINNY || d.algo == MNI_ALGO_SKINNY_TWO_PASS ||
         d.algo == MNI_ALGO_GEMV)) {
        int rc;
        if (try_skinny(d, &rc)) return rc;
        if (d.algo == MNI_ALGO_GEMV)
            return set_error(MNI_ERR_INVALID,
                             "sgemm: shape/layout not eligible for the decode product kernel (1 to 32 rows, one batch, row-major 16-byte "
                             "aligned B and C, N / 128 (N / 64 beyond 8 rows, with a 16-byte aligned A) a multiple of 8 that divides the "
                             "compute units, K a multiple of 512 (1024) times the compute units left per unit of columns)");
        if (d.algo == MNI_ALGO_SKINNY || d.algo == MNI_ALGO_SKINNY_TWO_PASS)
            return set_error(MNI_ERR_INVALID,
                             "sgemm: shape/layout not eligible for the skinny kernels "
                             "(needs min(M,N) <= 16 and 16-byte aligned unit-stride W)");
    }
    // A small N-contiguous B whose rows are not whole 16-byte pieces (N = 10 under a tall A) leaves the tile
    // kernel its element-wise loads of B; copied once into a K-contiguous layout it is read in 16-byte pieces
    // (65536 x 768 against [768, 10]: 77 us as given, 50 with the copy).  Not in the entry point that may not
    // allocate: the plan's own workspace has the one fixed block.
    // The same copy pays for a B of up to 16 MB whose N is off a multiple of 4 under a product of 1 to 6 GFLOP (too
    // small to be cut into a main part and a strip): its edge tiles would take the element-wise loop and the
    // launch would wait for them (1001 x 1003 x 999: 41 us as given, 24 with B given K-contiguous).
    const double flops = 2.0 * (double)d.M * (double)d.N * (double)d.K * (double)d.batch;
    const bool small_b = (d.B.row_stride % 4 != 0 || !aligned16(d.B.ptr) || (d.B.batch_count > 1 && d.B.batch_stride % 4 != 0)) && d.K % 4 == 0 &&
                         d.K * d.N * d.B.batch_count <= (1 << 18) && d.M * d.K * d.batch >= 16 * d.K * d.N * d.B.batch_count &&
                         d.M * d.K * d.batch >= (1LL << 20);
    const bool ragged_b = d.N % 4 != 0 && d.N >= 64 && d.M >= 64 && d.B.row_stride != 1 && flops >= 1e9 && flops < 6e9 &&
                          d.K * d.N * d.B.batch_count <= (1 << 22) && d.epilogue <= MNI_EPI_BIAS_GELU;
    // (and for an A given as its transpose whose M is off a multiple of 4: 1001 x 1003 x 999 transposed-A 56 us)
    const bool ragged_a = d.M % 4 != 0 && d.M >= 64 && d.N >= 64 && d.A.row_stride == 1 && d.A.col_stride != 1 && flops >= 1e9 && flops < 6e9 &&
                          d.M * d.K * d.A.batch_count <= (1 << 22) && d.epilogue <= MNI_EPI_BIAS_GELU;
    const bool pack_b = d.B.col_stride == 1 && d.N > 1 && (small_b || ragged_b);
    if (d.algo == MNI_ALGO_AUTO && d.split_k == 0 && !ctx().scratch && (pack_b || ragged_a)) {
        void *packed_a = nullptr, *packed_b = nullptr;
        mni_gemm_desc d2 = d;
        int rc = MNI_OK;
        if (pack_b) {
            rc = gemm_ws_alloc(&packed_b, (size_t)(d.K * d.N * d.B.batch_count) * sizeof(float));
            const int64_t shape[3] = {d.B.batch_count, d.N, d.K}, strides[3] = {d.B.batch_stride, d.B.col_stride, d.B.row_stride};
            if (rc == MNI_OK) rc = k_strided_copy((float *)packed_b, d.B.ptr, shape, strides, 3);
            d2.B.ptr = (const float *)packed_b;
            d2.B.row_stride = 1;
            d2.B.col_stride = d.K;
            d2.B.batch_stride = d.K * d.N;
        }
        if (rc == MNI_OK && ragged_a) {
            rc = gemm_ws_alloc(&packed_a, (size_t)(d.M * d.K * d.A.batch_count) * sizeof(float));
            const int64_t shape[3] = {d.A.batch_count, d.M, d.K}, strides[3] = {d.A.batch_stride, d.A.row_stride, d.A.col_stride};
            if (rc == MNI_OK) rc = k_strided_copy((float *)packed_a, d.A.ptr, shape, strides, 3);
            d2.A.ptr = (const float *)packed_a;
            d2.A.row_stride = d.K;
            d2.A.col_stride = 1;
            d2.A.batch_stride = d.M * d.K;
        }
        if (rc == MNI_OK) rc = run_mfma(d2);
        gemm_ws_free(packed_a);
        gemm_ws_free(packed_b);
        return rc;
    }
    return run_mfma(d);
}

// Two products that do not depend on each other (neither reads what the other writes; the outputs do not
// overlap).  One launch when run_mfma's plan for each of them alone is one workgroup per tile of the tile kernel and
// all of K, on 64 x 64 tiles both or on 128 x 128 tiles both.  Small tiles (batched products of about a tile per
// CU): together they give every SIMD a second wavefront and share one launch, one ramp-up and one tail.  Measured on
// 32 x (512 x 64 x 512) and its transposed twin: 13.4 + 13.6 us one after the other, 20.9 us together (64 batches of
// the first in one launch take the same 20.8).  Big tiles (the two gradients of a Linear layer): the second product's
// workgroups start where the first one's run out, so one drain and one fill of the machine go, and two products of
// one tile per CU each give every CU its second workgroup.  Measured on normally distributed operands, the pair
// issued back to back separately / as one launch, us: the gradients of [4096, 1024] . [1024, 4096] 489.6 / 473.0, of
// [4096, 4096] . [4096, 1024] (1024 tiles of K = 1024 behind 256 of K = 4096) 494.8 / 483.7, of 2048^3 259.8 / 245.4,
// [4096, 2048] . [2048, 2048] 484.2 / 474.1, [2048, 4096] . [4096, 1024] 257.1 / 250.6, [8192, 1024] . [1024, 4096]
// 943.2 / 922.3, 4096^3 1853.3 / 1849.4.  Otherwise one after the other.  Same kernel body and same order of every sum
// either way, so the results are those of the separate calls bit for bit.
int sgemm_pair(const mni_gemm_desc &d0, const mni_gemm_desc &d1, PairColsum *colsum) {
    if (colsum) colsum->done = false;
    MNI_TRY(ensure_init());
    MNI_TRY(validate(d0));
    MNI_TRY(validate(d1));
    DeviceCtx &c = ctx();
    const int cus = c.compute_units > 0 ? c.compute_units : 256;
    const mni_gemm_desc *ds[2] = {&d0, &d1};
    {
        // two products of a few thousand outputs each (sgemm would give each a launch of the tiny-product kernel)
        GemmLaunch t[2] = {};
        bool tiny = true;
        for (int i = 0; i < 2 && tiny; ++i) {
            const mni_gemm_desc &d = *ds[i];
            tiny = d.M > 0 && d.N > 0 && d.K > 0 && d.batch > 0 && d.algo == MNI_ALGO_AUTO && d.split_k == 0;
            if (tiny) {
                fill_launch(t[i], d);
                tiny = gemm_tiny_eligible(t[i]);
            }
        }
        if (tiny) {
            // (a thread per column walks the rows alone: only for a matrix a launch's worth of threads reads in a moment)
            const bool with_sums = colsum && colsum->src && colsum->out && colsum->rows > 0 && colsum->rows <= 256 && colsum->cols > 0 &&
                                   colsum->cols <= 4096 && colsum->rows * colsum->cols <= (1 << 16);
            MNI_TRY(launch_gemm_tiny_pair(t[0], t[1], with_sums ? colsum : nullptr));
            if (with_sums) colsum->done = true;
            return MNI_OK;
        }
    }
    PlanProbe plan[2];
    int64_t tiles = 0;
    bool pair = true, big = true;
    for (int i = 0; i < 2 && pair; ++i) {
        const mni_gemm_desc &d = *ds[i];
        // (min(M, N) <= 16 may go to the skinny kernels, which sgemm tries before run_mfma)
        pair = d.M > 16 && d.N > 16 && d.K > 0 && d.batch > 0 && d.algo == MNI_ALGO_AUTO && d.split_k == 0;
        if (!pair) break;
        {
            GemmLaunch t;
            fill_launch(t, d);
            if (gemm_tiny_eligible(t)) { pair = false; break; }  // sgemm computes those outright
        }
        MNI_TRY(run_mfma(d, &plan[i]));
        const bool whole = (plan[i].kind == PlanProbe::TILE || plan[i].kind == PlanProbe::TILE_FUSED_GELU) && plan[i].split == 1 &&
                           plan[i].bm == plan[i].bn;
        // 128 x 128 tiles: only products that sgemm would hand to run_mfma as they are (no batch to fold into the rows, no
        // ragged edge to cut off or operand to repack: every extent a multiple of 4)
        big = big && whole && plan[i].bm == 128 && d.batch == 1 && d.M % 4 == 0 && d.N % 4 == 0 && d.K % 4 == 0;
        pair = whole && (plan[i].bm == 64 ? plan[i].kind == PlanProbe::TILE : big);
        if (pair) tiles += (int64_t)plan[i].g.tiles_m * plan[i].g.tiles_n * plan[i].g.batch;
    }
    if (pair && plan[0].bm == plan[1].bm && gemm_mfma_pair_eligible(plan[0].amode, plan[0].bmode, plan[1].amode, plan[1].bmode)) {
        // 64 x 64: up to four workgroups fit a CU; beyond that a joint launch has nothing left to fill.  128 x 128: whatever
        // the tile counts (see above).
        if ((plan[0].bm == 64 && tiles <= 4LL * cus) || (plan[0].bm == 128 && big)) {
            // the caller's column sums ride along: workgroups behind the tiles that read the matrix once in the launch's tail
            // (4096 x 1024: two launches of 4.6 us each otherwise; the training step of a 4096 x 1024 -> 4096 -> 1024
            // network 1.512 -> 1.500 ms with both bias gradients taken this way)
            const bool with_sums = colsum && gemm_mfma_pair_takes_colsum(*colsum);
            MNI_TRY(launch_gemm_mfma_pair(plan[0].g, plan[0].amode, plan[0].bmode, plan[1].g, plan[1].amode, plan[1].bmode, plan[0].bm,
                                          with_sums ? colsum : nullptr));
            if (with_sums) colsum->done = true;
            return MNI_OK;
        }
    }
    MNI_TRY(sgemm(d0));
    return sgemm(d1);
}

}  // namespace mni

extern "C" int mni_rocm_sgemm_pair(const mni_gemm_desc *first, const mni_gemm_desc *second) {
    MNI_API_GUARD;
    if (!first || !second) return mni::set_error(MNI_ERR_INVALID, "sgemm_pair: null descriptor");
    return mni::sgemm_pair(*first, *second);
}

extern "C" int mni_rocm_sgemm(const mni_gemm_desc *desc) {
    MNI_API_GUARD;
    if (!desc) return mni::set_error(MNI_ERR_INVALID, "sgemm: null descriptor");
    return mni::sgemm(*desc);
}

extern "C" int64_t mni_rocm_sgemm_colsum_rows(int64_t M, int64_t batch) {
    // two strips per 128-row tile (the planner keeps 128-row tiles when strip sums are asked for)
    if (M <= 0 || batch <= 0) return 0;
    return batch * ((M + 127) / 128) * 2;
}

static int sgemm_timed_impl(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms, bool pairs);

extern "C" int mni_rocm_sgemm_timed(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms) {
    MNI_API_GUARD;
    return sgemm_timed_impl(descs, count, warmup, iters, avg_ms, false);
}

extern "C" int mni_rocm_sgemm_pair_timed(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms) {
    MNI_API_GUARD;
    if (count <= 0 || count % 2 != 0) return mni::set_error(MNI_ERR_INVALID, "sgemm_pair_timed: count must be a positive even number");
    return sgemm_timed_impl(descs, count / 2, warmup, iters, avg_ms, true);
}

// pairs: descs holds `count` pairs, each issued through sgemm_pair; the average is per pair.
static int sgemm_timed_impl(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms, bool pairs) {
    using namespace mni;
    if (!descs || count <= 0 || iters <= 0 || warmup < 0 || !avg_ms)
        return set_error(MNI_ERR_INVALID, "sgemm_timed: bad arguments");
    MNI_TRY(ensure_init());
    auto issue = [&](int i) { return pairs ? sgemm_pair(descs[2 * i], descs[2 * i + 1]) : sgemm(descs[i]); };
    int next = 0;
    for (int i = 0; i < warmup; ++i, next = (next + 1) % count) MNI_TRY(issue(next));
    hipEvent_t e0, e1;
    MNI_HIP_CHECK(hipEventCreate(&e0));
    MNI_HIP_CHECK(hipEventCreate(&e1));
    int rc = MNI_OK;
    hipError_t he = hipEventRecord(e0, ctx().stream);
    for (int i = 0; i < iters && rc == MNI_OK && he == hipSuccess; ++i, next = (next + 1) % count) rc = issue(next);
    if (he == hipSuccess) he = hipEventRecord(e1, ctx().stream);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != MNI_OK) return rc;
    if (he != hipSuccess) return set_error(MNI_ERR_HIP, "sgemm_timed: %s", hipGetErrorString(he));
    MNI_TRY(check_device_status("sgemm_timed"));
    *avg_ms = ms / (float)iters;
    return MNI_OK;
}
