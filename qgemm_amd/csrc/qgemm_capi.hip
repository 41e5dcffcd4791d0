// extern "C" layer of the library: argument checks, kernel choice, workspace,
// launches.  Declarations and the reference interfaces they replace are in
// include/qgemm.h.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <memory>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "aux_kernels.cuh"
#include "quant_kernels.cuh"
#include "selftest.cuh"
#include "variants.h"

using namespace qgemm;

#define QGEMM_EXPORT __attribute__((visibility("default")))

namespace {

// Scratch of the entry point that allocates nothing (qgemm_scaled_gemm_static): split-K partial planes,
// transposed block scales and transposed operands of one call.  One copy per device, held until the process
// ends; host code never uses the array's name as an address, only what hipGetSymbolAddress returned for the
// device that is current (static_scratch_locked).
constexpr size_t kStaticScratchBytes = QGEMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;

struct WsBlock {
    void *p = nullptr;
    size_t bytes = 0;
};

struct Context {
    std::mutex mu;
    bool ready = false;
    int device = -1;
    int num_cus = 256;
    // Workspace (split-K partial planes, transposed operands and scales, quantiser partials): one block for
    // the process.  A block that is outgrown is replaced and kept in `retired` until qgemm_shutdown: launches
    // already enqueued and graphs already captured keep pointing at live memory.  Calls on different streams
    // share the block and are ordered through ws_event: every call that used the workspace records it on its
    // stream when it has enqueued its launches, and a call on another stream waits for it first.
    WsBlock ws;
    std::vector<void *> retired;
    hipEvent_t ws_event = nullptr;
    hipStream_t ws_last_stream = nullptr;
    bool ws_event_recorded = false;
    bool ws_used_by_call = false;              // the running entry asked for the workspace
    bool static_call = false;                  // the running entry takes its workspace from the static scratch
    void *static_ptr[kMaxDevices] = {};        // device address of `scratch`, per device
    std::string force_config;   // name of a row of the variant tables, empty = heuristic (qgemm_force_config)
    long force_split = 0;       // 0 = heuristic
    long force_group_m = 0;     // 0 = default
#if QGEMM_DEBUG_BUILD
    long dbg_ptr = 0;           // measurement builds: device buffer for the kernels' time stamps (GemmArgs::dbg_cycles)
#endif
    long as_groups = 1;         // 0: a_scale always one K block per copy on the rows with two K groups (see run_nt)
    long small_tiles = 1;       // 0: 17 .. 256 rows never go to several row tiles of the skinny-M kernel in place of a K split
    long k_rot = -1;            // -1: rotated K start for at most 256 rows (see plan_nt), 0: never, n: steps per column tile
    long stagger = -1;          // -1: staggered start where it pays (4-byte C, three or more rounds), else microseconds per group
    long stagger_groups = 8;    // groups the workgroups of the first round start in
    long c_plain = -1;          // -1: the library decides; 0 / 1: non-temporal / ordinary stores for C
    long b_stream = -1;         // -1: the library decides; 0 / 1: B copies of the skinny-M kernel without / with the streaming hint
    long row_split = 1;         // 0: never run the rows (or columns) of a last, mostly empty round of 256 x 256 tiles as a second launch;
                                // 2 / 3: the rows / the columns always where the geometry allows it, whatever the estimate says
                                // (for measurements)
    long kmajor = 1;            // 0: K-major operands (NN, reference fp8 layout) always go through the transposes; 2: never
                                // where a K-major kernel fits the shape (for measurements and tests)
    std::string last_config;
};

Context g_ctx;

#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) return QGEMM_ERR_LAUNCH; \
    } while (0)

int static_scratch_locked(void **out);

int ensure_init_locked() {
    if (g_ctx.ready) return QGEMM_OK;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return QGEMM_ERR_NO_DEVICE;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    // The address of the static scratch on this device is looked up here, once, so that qgemm_scaled_gemm_static
    // finds it without a runtime call of its own; if the lookup fails only that entry is affected (it tries again
    // and reports the failure), every other entry works without the scratch.
    void *scratch_dev = nullptr;
    (void)static_scratch_locked(&scratch_dev);
    g_ctx.device = dev;
    g_ctx.num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    // tuning knobs, also reachable through qgemm_set_option
    if (const char *e = std::getenv("QGEMM_FORCE_CONFIG")) g_ctx.force_config = e;
    if (const char *e = std::getenv("QGEMM_GROUP_M")) g_ctx.force_group_m = std::atol(e);
    g_ctx.ready = true;
    return QGEMM_OK;
}

// Device address of the static scratch on the current device (looked up once per device).
int static_scratch_locked(void **out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return QGEMM_ERR_UNSUPPORTED;
    if (!g_ctx.static_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return QGEMM_ERR_LAUNCH;
        g_ctx.static_ptr[dev] = p;
    }
    *out = g_ctx.static_ptr[dev];
    return QGEMM_OK;
}

bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cap != hipStreamCaptureStatusNone;
}

// Workspace of `bytes` for a call enqueued on `stream`.
//   * qgemm_scaled_gemm_static: the static scratch; larger requests are an error, nothing is allocated.
//   * otherwise the library's block, grown when too small.  Growing allocates a new block and retires the old
//     one without freeing it (see Context).  While the stream is being captured into a graph nothing is
//     allocated and no event is waited for or recorded: a call that would have to grow the block fails with
//     QGEMM_ERR_ALLOC (the caller reserves the room before the capture, qgemm_reserve_workspace, or runs the
//     call once eagerly), and ordering replays against other users of the workspace is the caller's business.
int ensure_workspace_locked(size_t bytes, hipStream_t stream, void **out) {
    if (g_ctx.static_call) {
        if (bytes > kStaticScratchBytes) return QGEMM_ERR_SCRATCH_TOO_SMALL;
        return static_scratch_locked(out);
    }
    const bool capturing = stream_is_capturing(stream);
    if (bytes > g_ctx.ws.bytes) {
        if (capturing) return QGEMM_ERR_ALLOC;
        const size_t want = std::max({bytes, 2 * g_ctx.ws.bytes, (size_t)64 << 20});
        void *p = nullptr;
        if (hipMalloc(&p, want) != hipSuccess) {
            (void)hipGetLastError();
            return QGEMM_ERR_ALLOC;
        }
        if (g_ctx.ws.p) g_ctx.retired.push_back(g_ctx.ws.p);
        g_ctx.ws.p = p;
        g_ctx.ws.bytes = want;
    }
    if (!capturing) {
        if (g_ctx.ws_event_recorded && g_ctx.ws_last_stream != stream && !g_ctx.ws_used_by_call)
            HIP_TRY(hipStreamWaitEvent(stream, g_ctx.ws_event, 0));
        g_ctx.ws_used_by_call = true;
    }
    *out = g_ctx.ws.p;
    return QGEMM_OK;
}

// Around the body of every entry that may use the workspace: when it did, the end of its launches is recorded
// on its stream for the next user on another stream to wait for.
struct WorkspaceUse {
    hipStream_t stream;
    explicit WorkspaceUse(hipStream_t s) : stream(s) { g_ctx.ws_used_by_call = false; }
    ~WorkspaceUse() {
        if (!g_ctx.ws_used_by_call) return;
        g_ctx.ws_used_by_call = false;
        if (!g_ctx.ws_event && hipEventCreateWithFlags(&g_ctx.ws_event, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            g_ctx.ws_event = nullptr;
            return;
        }
        if (hipEventRecord(g_ctx.ws_event, stream) == hipSuccess) {
            g_ctx.ws_event_recorded = true;
            g_ctx.ws_last_stream = stream;
        } else {
            (void)hipGetLastError();
        }
    }
};

// kmaj: GemmCfg::KMAJ of the wanted family (0: both operands K-contiguous)
const Variant *table_for(int arith, bool block, int kmaj, int *count) {
    if (kmaj == 3) return (block && arith == AR_F8) ? variants_f8_block_tn(count) : nullptr;
    if (kmaj == 2) return block ? nullptr : (arith == AR_BF16 ? variants_bf16_nn(count) : (arith == AR_F16 ? variants_f16_nn(count) : nullptr));
    if (kmaj != 0) return nullptr;
    if (block) return arith == AR_F8 ? variants_f8_block(count) : (arith == AR_I8 ? variants_i8_block(count) : nullptr);
    switch (arith) {
        case AR_I8: return variants_i8(count);
        case AR_F8: return variants_f8(count);
        case AR_BF16: return variants_bf16(count);
        case AR_F16: return variants_f16(count);
    }
    return nullptr;
}

// Row `name` of a table, -1 when the family has no such row.
int row_by_name(const Variant *tab, int count, const std::string &name) {
    for (int i = 0; tab && i < count; ++i)
        if (name == tab[i].name) return i;
    return -1;
}
bool forced() { return !g_ctx.force_config.empty(); }

int arith_of(int in_dtype) {
    switch (in_dtype) {
        case QGEMM_DT_I8: return AR_I8;
        case QGEMM_DT_F8E4M3: return AR_F8;
        case QGEMM_DT_BF16: return AR_BF16;
        case QGEMM_DT_F16: return AR_F16;
    }
    return -1;
}

bool out_dtype_ok(int in_dtype, int out_dtype) {
    if (out_dtype == QGEMM_DT_F32 || out_dtype == QGEMM_DT_BF16 || out_dtype == QGEMM_DT_F16) return true;
    return out_dtype == QGEMM_DT_I32 && in_dtype == QGEMM_DT_I8;
}

struct NtProblem {
    int arith;
    bool block;
    const void *A, *B;
    void *C;
    size_t lda_bytes, ldb_bytes, ldc;   // ldc in elements; lda / ldb: stride between rows of m / n, or, for a
                                        // K-major operand (kmaj), between rows of k
    size_t M, N, Kbytes;
    int kmaj;                           // bit 0: A is stored K x M, bit 1: B is stored K x N
    const float *as, *bs;
    uint32_t as_ms, as_ks, bs_ns, bs_ks;
    int out_dtype, per_matrix, split_k;
};

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

size_t ksteps_of(const NtProblem &q) { return (q.Kbytes + 127) / 128; }      // the last one may be partial

// Shapes the MFMA kernel takes (pointer alignment is checked separately); everything else goes to the any-shape
// kernel.  K is a whole number of 16-byte chunks (the unit of a copy); a last K step of fewer than 128 bytes is
// filled up with zeros on the way into LDS (GemmArgs::k_tail), which the reference's dispatch covers with its
// 64- and 32-wide K tiles (hip_mix_gemm_kernel.cpp:442-463).
bool mfma_shape_ok(const NtProblem &q) {
    const size_t es = (q.arith == AR_BF16 || q.arith == AR_F16) ? 2 : 1, krows = q.Kbytes / es;
    // 32-bit buffer offsets: 256 tile rows of a K-contiguous operand (plus the 3072 bytes by which the solo kernels
    // shift their descriptors), every k row of a K-major one.  With a partial last K step the lanes past the end of
    // a row mark their offsets with bit 31: every valid offset then has to stay below 2^31.
    const size_t lim = (size_t)1 << (q.Kbytes % 128 ? 31 : 32);
    const bool a_ok = (q.kmaj & 1) ? (krows * q.lda_bytes < ((size_t)1 << 32) && q.lda_bytes >= q.M * es)
                                   : q.lda_bytes * 256 + 4096 < lim;
    const bool b_ok = (q.kmaj & 2) ? (krows * q.ldb_bytes < ((size_t)1 << 32) && q.ldb_bytes >= q.N * es)
                                   : q.ldb_bytes * 256 + 4096 < lim;
    // block scales: the kernel addresses a_scale with 32-bit byte offsets ((kb * as_ks + m) * 4)
    const bool s_ok = !q.block || ((q.Kbytes + 127) / 128) * std::max<size_t>(q.M, q.as_ks) * 4 < ((size_t)1 << 32);
    return q.Kbytes % 16 == 0 && q.Kbytes > 0 && q.lda_bytes % 16 == 0 && q.ldb_bytes % 16 == 0 && a_ok && b_ok && s_ok &&
           q.M < ((size_t)1 << 31) && q.N < ((size_t)1 << 31) && q.ldc < ((size_t)1 << 32);
}

// Which tile, and how many K slices.
//
// M > 64: a cost estimate over the tiles worth having there (256 x 256 solo, 128 x 128 in two forms, 64 x 128, 128 x 32) and
// 1 / 2 / 4 / 8 K slices.  Workgroups run in rounds of CUs x (workgroups that fit a CU); a round costs
// (K steps x time per step + a fixed prologue / epilogue), a last partial round that leaves a 128 x 128
// workgroup alone on its CU runs its steps faster, and a K split pays a second launch plus the traffic of the
// partial planes.  The times per 128-byte K step were read off a sweep of every variant over square and oblong
// shapes from 1024 to 8192 (fp8 and bf16 agree per step; block scales have figures of their own): 1.25 us for the
// 256 x 256 tile (one per CU), 0.85 us for 128 x 128 with two per CU and 0.66 us alone, 0.43 us for the 128 x 128
// row with two K groups (one per CU: it only wins where there are no more tiles than CUs; 2048 x 2048 x 2048 / 8192
// 12.1 / 32.5 us), 0.52 us for 64 x 128 and 0.27 us for its row with two K groups (512 x 4096 x 4096 13.5 us, two
// rounds of 64 steps 44 us), 0.39 us for 128 x 32; for 256 x 128 with its copying waves 0.71 us with every CU at work,
// which is what the 256 x 256 tile needs per flop, and 0.58 us with 160 - 224 tiles (0.93 / 0.76 with block scales),
// plus 6 us around a round (2048 x 4096 x 4096 29.3 us, 1024 x 8192 x 8192 50.8, 1536 x 4096 x 4096 25.2,
// 768 x 7168 x 2048 14.8; it wins where its tiles make one round of CUs and the 256 x 256 tiles would leave half of
// them idle: 6 - 17 % over the two-stage 128 x 128 row there, with block scales up to 24 %).
// 192 x 256 (8-wave solo schedule) for row counts whose 256-row tiles leave a round partly empty: 1.03 us a step in a
// full round, 0.97 in a partly filled one (1.27 / 1.18 with block scales), 6 us around a round (3072 x 4096 x 4096 fp8
// 43.7 us against 47.5 on 192 tiles of 256 x 256, 2560 rows 37.7 against 42.8, 1536 x 7168 x 2048 23.3 against 26.8,
// bf16 1152 x 8192 x 4096 64.6 against 78.3).  Full rounds refitted on 36 large shapes per type with every large row
// forced (they had been priced at 1.10 / 1.30, 7 - 10 % above what was measured): shapes whose 192-row tiles make
// whole rounds now run on them in one launch instead of a 256 x 256 launch and a rest (6144^3: 768 tiles, three
// rounds; fp8 165.9 -> 163.7 us, block scales 206.9 -> 198.1, bf16 327.4 -> 318.5; over the 71 of 1440 grid shapes
// whose plan changed the new plan is 3.0 % faster on average, at worst 1.6 % slower).
// A K split adds 4 us and the partial planes at 3 TB/s.
//
// M <= 64 (bandwidth-bound, B is streamed once): the largest tile that still gives three quarters of the CUs a
// workgroup, else the shortest tile that covers the rows; narrow tiles instead of a K split.  (65 .. 128 rows go
// through the estimate as well: it keeps the 128 x 32 tile for the short K of config 5 and prefers a 128 x 128 tile
// with a K split where K is long, 128 x 8192 x 8192 bf16 38 against 48 us.)
struct TileModel {
    int bm, bn, per_cu;
    double step_shared, step_alone, fixed;     // microseconds
    bool kgroups;                              // the row of this tile with two K groups per workgroup (GemmCfg::KG)
    // the same with 128-block scales (fp8): the fold costs the 8-wave 256 x 256 kernel a tenth, the simple pipeline
    // more (its block-scaled rows have two stages, so more workgroups share a CU), the K-group rows most
    int blk_per_cu;
    double blk_shared, blk_alone;
};
// (block scales, graph replays: 256 x 256 2048 x 4608 x 7168 77 us, 1536 x 7168 x 2048 27.6; 128 x 128 1024 x 7168 x 2048 25.9,
// 1024 x 4608 x 7168 75.0; 64 x 128 1024 x 4608 x 7168 69.9, 512 x 4608 x 7168 47.8; K groups 128 x 128 2048 x 2048 x 2048 /
// 8192 14 / 43, 64 x 128 512 x 4096 x 4096 18, and with the a_scale values of four K blocks per copy (GemmArgs::as_groups)
// 38 - 41 and 15.3; 128 x 32 256 x 7168 x 2048 12.9)
const TileModel kTileModels[] = {{256, 256, 1, 1.25, 1.25, 4.0, false, 1, 1.40, 1.40}, {128, 128, 2, 0.85, 0.66, 2.0, false, 2, 1.32, 1.04},
                                 {128, 128, 1, 0.43, 0.43, 4.5, true, 1, 0.50, 0.50},  {64, 128, 1, 0.52, 0.52, 1.5, false, 3, 1.21, 0.83},
                                 {64, 128, 1, 0.27, 0.27, 4.5, true, 1, 0.34, 0.34},   {128, 32, 1, 0.39, 0.39, 1.0, false, 2, 0.74, 0.60},
                                 {256, 128, 1, 0.71, 0.58, 6.0, false, 1, 0.93, 0.76}, {192, 256, 1, 1.03, 0.97, 6.0, false, 1, 1.27, 1.18}};
// rows with two K groups: two sets of computing waves on a tile that otherwise has one (one workgroup per CU)
bool is_kgroup_row(const Variant &v) { return v.kgroups == 2; }

int choose_by_cost(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int cus, bool may_split,
                   uint32_t *nsplit_out, double *cost_out = nullptr) {
    int best = -1;
    double best_t = 0;
    for (const TileModel &tm : kTileModels) {
        int vi = -1;
        for (int i = 0; i < count; ++i)
            if (tab[i].auto_ok && tab[i].bm == tm.bm && tab[i].bn == tm.bn && is_kgroup_row(tab[i]) == tm.kgroups) vi = i;
        if (vi < 0) continue;
        const size_t tiles = ((M + tm.bm - 1) / tm.bm) * ((N + tm.bn - 1) / tm.bn);
        for (uint32_t ns = 1; ns <= 8; ns *= 2) {
            if (ns > 1 && (!may_split || ksteps / ns < 4)) break;
            const size_t wgs = tiles * ns, slots = (size_t)cus * (block ? tm.blk_per_cu : tm.per_cu), steps = (ksteps + ns - 1) / ns;
            const size_t full = wgs / slots, rem = wgs % slots;
            const double shared = block ? tm.blk_shared : tm.step_shared, alone = block ? tm.blk_alone : tm.step_alone;
            double t = (double)full * (steps * shared + tm.fixed);
            if (rem) t += steps * (rem <= (size_t)cus ? alone : shared) + tm.fixed;
            if (ns > 1) t += 4.0 + (double)M * N * 4.0 * (ns + 1) / 3.0e6;
            if (best < 0 || t < best_t) {
                best = vi;
                best_t = t;
                *nsplit_out = ns;
            }
        }
    }
    if (cost_out) *cost_out = best_t;
    return best;
}

int choose_tile(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int kmaj, int cus,
                bool may_split, uint32_t *nsplit_out);
size_t rows_for_full_rounds(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int cus,
                            double t_single, double *t_split = nullptr, size_t *padding = nullptr);
size_t cols_for_full_rounds(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int cus,
                            double t_single, double *t_split = nullptr, size_t *padding = nullptr, bool whatever_the_estimate = false);

// The skinny-M kernel (gemm_skinny.cuh: the K split inside the workgroup, eight waves each on every eighth K step)
// takes over from the narrow simple-pipeline tiles where it is faster: one row tile (M <= 128), a strip of 32
// columns per workgroup as the tile choice below would have it, and enough K steps for the eight waves (two each;
// one each is enough up to 16 rows).  Graph replays over rotated B, fp8, microseconds per launch, narrow tile
// against skinny kernel: 16 x 7168 x 2048 7.6 / 5.4, 64 x 7168 x 2048 9.0 / 6.7, 128 x 7168 x 2048 11.0 / 8.2,
// 16 x 7168 x 8192 24.6 / 15.2, 32 x 4096 x 4096 12.7 / 8.3, 128 x 4096 x 4096 18.3 / 12.5, 16 x 1024 x 1024
// 5.6 / 3.1; with K = 1024 and more than 16 rows or K = 512 the narrow tiles stay ahead (64 x 8192 x 1024 5.0 / 5.2,
// 128 x 7168 x 512 4.6 / 6.0).  The same rule serves block scales (B resident: 16 x 7168 x 2048 10.8 / 6.6,
// 128 x 7168 x 2048 15.7 / 9.5).
// A K split across workgroups on top pays only where the strips leave at least half of the CUs without work and K is
// long: a workgroup moves its strip of B and its rows of A at about 45 GB/s, a split divides that time and adds a
// reduction launch of about 4.5 us.  B out of HBM, microseconds per launch, one workgroup per strip against the split
// this estimate picks: 16 x 4096 x 14336 fp8 20.6 / 17.2 (two slices), bf16 37.1 / 26.9; 64 x 4096 x 14336 27.3 / 22.7,
// bf16 53.7 / 37.2; 64 x 2048 x 8192 15.2 / 11.3 (four slices), bf16 26.8 / 14.7; no split for 16 x 4096 x 4096 (7.6
// against 9.5 with two slices) and none where the strips fill the CUs (16 x 8192 x 8192 15.2 against 18.8).
// kmaj: the table is a K-major family, which has no narrow tiles: the estimate then serves every M
int choose_variant(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int kmaj, int cus,
                   bool may_split, uint32_t *nsplit_out) {
    const int vi = choose_tile(tab, count, M, N, ksteps, block, kmaj, cus, may_split, nsplit_out);
    // The same kernel on 64 x 64 tiles: shapes with several row tiles whose 64 x 64 tiles fit one
    // round of CUs and give most of them work, 16 K steps or more.  Against whatever the estimate picks (narrow
    // tiles, K-group tiles with a K split) it is 13 - 33 % faster over 512 .. 2048 rows x 256 .. 3000 columns x 2 .. 8 KiB
    // of K (fp16 1024^3 7.3 -> 6.3 us, fp8 1000 x 1000 x 4096 13.1 -> 8.8), slower only with 8 K steps (one per wave)
    // or with 64 tiles and 64 K steps; beyond 64 K steps the tiles with a K split across workgroups catch up
    // (bf16 256 x 2048 x 7168, 112 steps: 18.9 against 22.9 us).  With block scales the gain is larger, the small tiles
    // of the simple pipeline being slower there: 512 x 2048 x 4096 18.3 -> 11.7 us, 256 x 4096 x 4096 17.8 -> 11.8.
    // From 65 rows on: with two row tiles a workgroup pulls half of A (an L2 hit, but through its CU's load path) next
    // to twice the strip of B, 256 KiB instead of 320 KiB at 128 x 7168 x 2048, the smallest sum a tile of that area
    // has (config 5 at M = 128, B out of HBM: 8.9 -> 8.3 us; M = 64 stays on 32-column strips, 6.8 us).
    // 17 .. 256 rows against few columns, 32 .. 48 K steps: tiles of 16 x 32, 32 x 32, 64 x 32 or 64 x 64 on the skinny-M kernel,
    // several over the rows, whichever fills at most one round of CUs with the least to move: a workgroup moves its rows
    // of A at about 100 GB/s (L2 hits) and its strip of B at about 45 GB/s (out of memory), all of them together about
    // 12 TB/s (the row tiles of a strip share it in the L2s); constants fitted on 90 shapes x 4 tiles x (one B, B in
    // rotation through 600 MB).  That beats a taller tile with a K split across workgroups (a second launch of 4.5 us)
    // and the 64 x 64 form where smaller tiles still fit a round.  Graph replays, us, one B / B in rotation through
    // 600 MB, what the rules below took against this: 128 x 1024 x 4096 fp8 10.0 / 10.7 (128 x 32, four slices) ->
    // 5.4 / 6.6 (32 x 32), 96 x 2048 x 4096 8.8 / 11.3 (64 x 64) -> 6.5 / 7.9, 128 x 2048 x 4096 8.8 / 11.8 -> 7.6 / 9.1
    // (64 x 32), 130 x 1536 x 6144 12.8 / 13.7 -> 10.0 / 11.0; bf16 the same at the same bytes of K, block scales
    // 128 x 2048 x 4096 10.5 / 13.0 -> 8.7 / 9.7.  From 56 K steps on the small tiles still win with B resident
    // (160 x 2048 x 7168 13.5 -> 12.2) but lose with B streamed (14.9 -> 17.7: fewer, longer streams), so the K split
    // stays there; block scales only up to 32 K steps (their fold makes the longer loops of the small tiles slower).
    // 24 .. 256 rows x 1024 .. 7168 columns x 4 and 6 KiB of K, fp8, 90 shapes: 13 % less time with B resident, 9.5 % with B
    // streamed, two shapes more than 3 % slower (7 % at worst); 64 x 1024 x 4096 fp8 7.7 / 8.5 (64 x 32, four slices) ->
    // 4.7 / 5.6 (16 x 32).  A smaller tile has to be estimated 3 % ahead of a larger one.
    if (vi >= 0 && !kmaj && g_ctx.small_tiles && M > 16 && M <= 256 && ksteps >= 32 && ksteps <= (block ? 32u : 48u)) {
        int best = -1;
        double best_t = 0;
        static const int kSmall[4][2] = {{64, 64}, {64, 32}, {32, 32}, {16, 32}};       // (a smaller tile has to be 3 % ahead)
        for (const auto &bt : kSmall)
            for (int i = 0; i < count; ++i) {
                const Variant &v = tab[i];
                if (v.kgroups != 8 || v.bm != bt[0] || v.bn != bt[1]) continue;
                const size_t tiles = ((M + v.bm - 1) / v.bm) * ((N + v.bn - 1) / v.bn);
                if (tiles > (size_t)cus) continue;
                const double kb = ksteps * 128.0;
                const double t = std::max(v.bm * kb / 100.0e3 + v.bn * kb / 45.0e3, tiles * (v.bm + v.bn) * kb / 12.0e6);
                if (best < 0 || t < 0.97 * best_t) {
                    best = i;
                    best_t = t;
                }
            }
        if (best >= 0) {
            *nsplit_out = 1;
            return best;
        }
    }
    if (vi >= 0 && !kmaj && M > 64 && ksteps >= 16 && ksteps <= 64) {
        const size_t t64 = ((M + 63) / 64) * ((N + 63) / 64);
        // (with more than 48 K steps and weights streamed out of memory, half a round of such tiles is behind a wider tile
        // with a K split, which has twice the streams: 256 x 2048 x 8192 fp8 18.3 against 16.1 us, 13.5 against 13.8 with
        // B resident; from 160 tiles on the 64 x 64 form is ahead either way)
        if (t64 <= (size_t)cus && ((t64 >= 128 && (ksteps <= 48 || t64 >= 160)) || (t64 >= 64 && ksteps <= 32)))
            for (int i = 0; i < count; ++i)
                if (tab[i].kgroups == 8 && tab[i].bm == 64 && tab[i].bn == 64) {
                    *nsplit_out = 1;
                    return i;
                }
    }
    if (vi < 0 || kmaj || M > 128) return vi;
    const size_t strips = (N + 31) / 32;
    // Up to 32 rows against so few columns that 32-column strips leave half of the CUs idle, 32 .. 112 K steps: strips of
    // 16 columns, one workgroup each and no K split across workgroups (which costs a second launch).  Graph replays, us,
    // one B / B in rotation through 600 MB, fp8 (bf16 the same at the same bytes of K): 16 x 4096 x 14336 14.7 / 15.8
    // (32-column strips, two slices) -> 12.6 / 13.0 (vendor library 12.7 / 14.7), 16 x 4096 x 8192 11.5 / 12.1 -> 9.4 / 9.0,
    // 16 x 2048 x 8192 7.2 / 9.6 -> 5.6 / 7.7, 32 x 4096 x 14336 16.2 / 18.1 -> 15.8 / 16.6; from 128 K steps on the split is
    // ahead (16 x 2048 x 16384 10.2 / 11.0 against 12.2 / 13.2), and with 64 rows the two are level or the split ahead.
    // With fewer than 192 such strips (N < 3072) only up to 16 rows and 64 K steps: beyond that the streams are too few
    // and too long, and the split is 4 - 50 % ahead with B streamed (32 x 1024 x 14336 9.5 against 14.7 us).  Not with block
    // scales (3 - 30 % slower throughout).
    const size_t strips16 = (N + 15) / 16;
    if (g_ctx.small_tiles && !block && M <= 32 && ksteps >= 32 && ksteps <= 112 && strips * 2 <= (size_t)cus && strips16 <= (size_t)cus &&
        (strips16 >= 192 || (M <= 16 && ksteps <= 64)))
        for (int i = 0; i < count; ++i)
            if (tab[i].kgroups == 8 && tab[i].bn == 16 && (size_t)tab[i].bm >= M) {     // (rows of the table in ascending height)
                *nsplit_out = 1;
                return i;
            }
    // 17 .. 64 rows against so many columns that the 32-column strips need a second round of CUs while 64-column
    // strips fit in one: the 64 x 64 form (half the strips, each row of A fetched half as often).  B out of HBM:
    // 64 x 14336 x 4096 bf16 34.3 -> 26.7 us, fp8 20.4 -> 17.0; 48 rows 33.4 -> 27.4 and 19.4 -> 16.5; 32 rows bf16
    // 26.4 -> 23.5, 32 x 14336 x 8192 49.7 -> 41.2, 24 x 11008 x 4096 24.4 -> 22.5, 32 x 12288 x 2048 fp8 10.4 -> 9.1
    // (up to 16 rows the two are level).
    if (M > 16 && M <= 64 && ksteps >= 16 && strips > (size_t)cus && (N + 63) / 64 <= (size_t)cus)
        for (int i = 0; i < count; ++i)
            if (tab[i].kgroups == 8 && tab[i].bm == 64 && tab[i].bn == 64) {
                *nsplit_out = 1;
                return i;
            }
    // 65 .. 128 rows come out of the estimate above, whose times per step are those of operands that sit in the caches;
    // with B streamed out of memory the skinny-M kernel is ahead wherever its strips fit one round of CUs and K is
    // not long enough for a K split to pay (128 x 7168 x 2048 bf16 17.8 -> 13.6 us, 128 x 8192 x 8192 fp8 26.9 -> 24.8)
    const bool mid_rows = M > 64 && strips <= (size_t)cus && ksteps >= 16 && ksteps <= 64;
    // (up to 64 rows the choice above takes a wide tile with a K split where 32-column tiles of its height would need
    // more than two rounds; up to two rounds of strips the skinny-M kernel is ahead of that too: 32 x 14336 x 4096 fp8
    // 24.6 -> 17.2 us, bf16 36.4 -> 29.7; with 896 strips the wide tiles stay, 32 x 28672 x 8192 46.8 against 55.1)
    const bool few_strips = M <= 64 && strips <= 2 * (size_t)cus && ksteps >= 16;
    if (!mid_rows && !few_strips && (tab[vi].bn != 32 || tab[vi].kgroups != 1)) return vi;
    if (ksteps < 8 || (ksteps < 16 && M > 16)) return vi;
    for (int i = 0; i < count; ++i)
        if (tab[i].kgroups == 8 && tab[i].bn == 32 && (size_t)tab[i].bm >= M) {        // (rows of the table in ascending height)
            *nsplit_out = 1;
            if (may_split && strips * 2 <= (size_t)cus) {
                const double t_one = (double)(32 + tab[i].bm) * ksteps * 128.0 / 45.0e3;     // us, one workgroup per strip
                double best = t_one;
                for (uint32_t ns = 2; ns <= 8 && strips * ns <= (size_t)cus && ksteps / ns >= 8; ++ns) {
                    const double t = t_one / ns + 4.5;
                    if (t < best) {
                        best = t;
                        *nsplit_out = ns;
                    }
                }
            }
            return i;
        }
    return vi;
}

int choose_tile(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int kmaj, int cus,
                bool may_split, uint32_t *nsplit_out) {
    *nsplit_out = 0;                                       // 0: no opinion, plan_nt decides
    if (M > 64 || kmaj) {
        int vi = choose_by_cost(tab, count, M, N, ksteps, block, cus, may_split, nsplit_out);
        if (vi >= 0) {
            // 256 x 256, int8 and 16-bit types: the 8-wave form needs fewer cycles per tile, the 4-wave form a third
            // fewer LDS reads.  With at least one full round of CUs the part runs at its power limit and the 4-wave
            // form wins by 2 - 3 % (higher clock; level in the partly filled rounds of such shapes); with fewer
            // tiles than CUs the clock is not what limits and the 8-wave form wins by 1 - 5 %.  (fp8 per-matrix:
            // the 4-wave form either way; block scales: 8 waves.)
            const Variant &v = tab[vi];
            const size_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
            if (v.bm == 256 && v.bn == 256 && v.threads == 512 && !block && kmaj == 0 && *nsplit_out <= 1 && tiles >= (size_t)cus)
                for (int i = 0; i < count; ++i)
                    if (tab[i].bm == 256 && tab[i].bn == 256 && tab[i].threads == 256 && tab[i].lds_bytes == v.lds_bytes &&
                        !std::strcmp(tab[i].name, "256x256_w2x2_solo"))
                        vi = i;
            return vi;
        }
        *nsplit_out = 0;
    }
    const size_t m16 = std::max<size_t>(16, (M + 15) / 16 * 16);
    const size_t target = std::min<size_t>(m16, 128);   // shorter tiles would stream B more than once
    int best = -1;
    size_t best_area = 0;
    for (int i = 0; i < count; ++i) {
        if (!tab[i].auto_ok || is_kgroup_row(tab[i]) || (size_t)tab[i].bm > m16 || (size_t)tab[i].bm < target) continue;
        const size_t tiles = ((M + tab[i].bm - 1) / tab[i].bm) * ((N + tab[i].bn - 1) / tab[i].bn);
        const size_t area = (size_t)tab[i].bm * tab[i].bn;
        if (tiles * 4 >= (size_t)cus * 3 && area > best_area) {     // at least three quarters of the CUs get a tile
            best = i;
            best_area = area;
        }
    }
    if (best >= 0) return best;
    // Nothing fills the CUs: 16 x 32 tiles, several over the rows, while they make at most two rounds (B is read once
    // per 16 rows then, out of the L2: 48 x 4096 x 4096 fp8 10.5 us against 14.7 with a 64 x 128 tile and a K split);
    // else the shortest tile that covers the rows, the narrowest of that height.
    for (int i = 0; i < count; ++i)
        if (tab[i].auto_ok && tab[i].bm == 16 && tab[i].bn == 32 && ((M + 15) / 16) * ((N + 31) / 32) <= 2 * (size_t)cus) return i;
    for (int i = 0; i < count; ++i) {
        if (!tab[i].auto_ok || is_kgroup_row(tab[i]) || (size_t)tab[i].bm < target) continue;
        if (best < 0 || tab[i].bm < tab[best].bm || (tab[i].bm == tab[best].bm && tab[i].bn < tab[best].bn)) best = i;
    }
    return best;
}

// Should the problem run with these operands read K-major, as they are stored (strides between k rows given)?
// Yes when the shape fits and the estimate for the K-major family beats the K-contiguous kernel plus the transpose
// launches in front of it (4 us per operand and the matrix read and written at 5.5 TB/s; block scales 2048^3 in the
// reference's layout: 23.3 us as stored, 29.3 us behind two transposes; 1024 x 4096 x 4096: 39.9 against 37.2).
// The simple-pipeline rows pay 15 % on top of the estimate for their transposing reads.  The 256 x 128 row with
// copying waves needs per K step what its K-contiguous form needs, and is taken up to 2.5 % above the other route's
// estimate (which counts a row split where the K-contiguous plan would make one, and runs low for one round of
// 256 x 256 tiles behind transposes).  Measured, as stored against through the transposes, us: fp8_mm 4096^3
// 65.3 / 73.9, 2048 x 4096 x 4096 35.0 / 46.9, 3072 x 8192 x 4096 102.8 / 110.4, bf16 with B stored K x N 4096^3
// 101.4 / 109.6, 2048 x 8192 x 8192 194.6 / 223.3, 2048 x 4096 x 4096 52.2 / 68.2; the largest shapes keep the
// transposes and the 256 x 256 tile: config 4 in the reference's storage 207.8 / 194.6, 8192^3 506.6 / 465.2 (fp8_mm)
// and 786.0 / 742.4 (bf16), 6144^3 240.3 / 229.6 and 356.7 / 348.6.  Over 19 shapes the ratio of the two estimates is
// within 4 % of the measured ratio on 15 and the choice is the faster route on all but bf16 3072 x 4096 x 4096 (4 %).
bool kmajor_problem_ok(NtProblem q, int kmaj, size_t lda_bytes, size_t ldb_bytes) {
    if (!g_ctx.kmajor) return false;
    q.kmaj = kmaj;
    q.lda_bytes = lda_bytes;
    q.ldb_bytes = ldb_bytes;
    if (!mfma_shape_ok(q)) return false;
    int count = 0, count_km = 0;
    const Variant *tab = table_for(q.arith, q.block, 0, &count), *tab_km = table_for(q.arith, q.block, kmaj, &count_km);
    if (!tab || !tab_km) return false;
    if (forced()) return row_by_name(tab_km, count_km, g_ctx.force_config) >= 0;   // a forced row: as stored where the K-major family has it
    if (g_ctx.kmajor == 2) return true;                                        // measurements: as stored wherever possible
    const size_t ksteps = ksteps_of(q);
    const bool may_split = q.split_k == 0;
    uint32_t ns = 0;
    double t_km = 0, t_nt = 8.0;                    // a skinny K-contiguous launch: about 8 us
    const int vk = choose_by_cost(tab_km, count_km, q.M, q.N, ksteps, q.block, g_ctx.num_cus, may_split, &ns, &t_km);
    if (vk < 0) return false;
    if (q.M > 128 && choose_by_cost(tab, count, q.M, q.N, ksteps, q.block, g_ctx.num_cus, may_split, &ns, &t_nt) < 0)
        return false;
    if (q.M > 128 && may_split) {                    // (the K-contiguous route may split the rows into two launches)
        double t_single = 0, t_split = 0;
        uint32_t ns1 = 0;
        if (choose_by_cost(tab, count, q.M, q.N, ksteps, q.block, g_ctx.num_cus, false, &ns1, &t_single) >= 0) {
            if (rows_for_full_rounds(tab, count, q.M, q.N, ksteps, q.block, g_ctx.num_cus, t_single, &t_split) && t_split < t_nt)
                t_nt = t_split;
            if (cols_for_full_rounds(tab, count, q.M, q.N, ksteps, q.block, g_ctx.num_cus, t_single, &t_split) && t_split < t_nt)
                t_nt = t_split;
        }
    }
    const double kbytes = (double)q.Kbytes;         // K * element size
    t_nt += 1.0;                                     // a transpose launch per operand: 4 us and the matrix read and written
    if (kmaj & 1) t_nt += 4.0 + 2.0 * (double)q.M * kbytes / 5.5e6;
    if (kmaj & 2) t_nt += 4.0 + 2.0 * (double)q.N * kbytes / 5.5e6;
    return tab_km[vk].copy_waves ? t_km <= 1.025 * t_nt : 1.15 * t_km <= t_nt;
}

struct Plan {
    const Variant *v = nullptr;
    GemmArgs a;
    size_t tiles = 0;
    size_t split_bytes = 0;   // workspace the K split needs (0 when not split)
    // Row split: this plan covers rows [0, m_main) of the problem and `rest` the rows below, as a second launch
    // with a tile of its own (m_main = 0: no split, the plan covers everything).
    size_t m_main = 0;
    // Column split, the same along N: columns [0, n_main) here, the columns to the right in `rest` (never both splits)
    size_t n_main = 0;
    std::unique_ptr<Plan> rest;
};

// elements the tiles of a launch compute beyond the M x N asked for
size_t padded_area(size_t bm, size_t bn, size_t M, size_t N) {
    return ((M + bm - 1) / bm * bm) * ((N + bn - 1) / bn * bn) - M * N;
}

// Rows of the problem that 256 x 256 tiles should take when such tiles do not fill the last round of CUs.
// 576 tiles on 256 CUs are 2.25 rounds and cost three: the rows of the two full rounds go to one launch, and the
// rows below to whatever the tile choice likes best for them (smaller tiles, which fill the CUs; the skinny-M
// kernel for up to 128 rows).  Also where a single launch would rather take smaller tiles for everything
// (5000 x 4096 x 7168: 1.25 rounds of 256 x 256 tiles; fp8 148 us as one launch of 128 x 128 tiles, 113 us as 4096 rows
// of 256 x 256 tiles and 904 rows of 128 x 128 ones; 7000 x 7168 x 2048: 106 -> 93 us with the last 88 rows on the
// skinny-M kernel).  Returns 0 for "do not split": when the estimate of the two launches (plus 6 us for the
// second) is not at least 2.5 % below the estimate t_single of the one (config 4 with block scales: estimate
// 160.5 against 164.8 us, 2.6 %; measured 170.9 - 172.5 against 175.1 - 176.9 us in three interleaved runs).
size_t rows_for_full_rounds(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int cus,
                            double t_single, double *t_split, size_t *padding) {
    if (!g_ctx.row_split) return 0;
    const size_t tn = (N + 255) / 256, tiles = ((M + 255) / 256) * tn, full = tiles / cus;
    if (full == 0 || tiles % cus == 0) return 0;
    const size_t m_main = (full * cus / tn) * 256;
    if (m_main == 0 || m_main >= M) return 0;
    uint32_t ns = 0;
    double t_main = 0, t_rest = 0;
    const int vm = choose_by_cost(tab, count, m_main, N, ksteps, block, cus, false, &ns, &t_main);
    if (vm < 0 || tab[vm].bm != 256 || tab[vm].bn != 256) return 0;
    size_t pad = padded_area(256, 256, m_main, N);
    if (M - m_main > 128) {
        const int vr = choose_by_cost(tab, count, M - m_main, N, ksteps, block, cus, false, &ns, &t_rest);
        if (vr < 0) return 0;
        pad += padded_area(tab[vr].bm, tab[vr].bn, M - m_main, N);
    } else {
        t_rest = 5.0 + (double)N * ksteps * 128.0 / 4.0e6;      // B streamed once, about 4 TB/s
    }
    if (t_split) *t_split = t_main + t_rest + 6.0;
    if (padding) *padding = pad;
    if (g_ctx.row_split == 2) return m_main;
    return t_main + t_rest + 6.0 < 0.975 * t_single ? m_main : 0;
}

// The same along N, for shapes whose row tiles do not divide the full rounds but whose column tiles do:
// 4096 x 14336 x 4096 is 16 x 56 tiles, 3.5 rounds; 13 of its 16 row tiles are 2.84 rounds and still cost three, while
// 48 of its 56 column tiles are exactly three, and the 4096 x 2048 to their right fill a round of smaller tiles.
// Returns the columns of the first launch (a multiple of 256, so the right part starts on a 128-block of b_scale).
size_t cols_for_full_rounds(const Variant *tab, int count, size_t M, size_t N, size_t ksteps, bool block, int cus,
                            double t_single, double *t_split, size_t *padding, bool whatever_the_estimate) {
    if (!g_ctx.row_split) return 0;
    const size_t tm = (M + 255) / 256, tiles = tm * ((N + 255) / 256), full = tiles / cus;
    if (full == 0 || tiles % cus == 0) return 0;
    const size_t n_main = (full * cus / tm) * 256;
    if (n_main == 0 || n_main >= N) return 0;
    uint32_t ns = 0;
    double t_main = 0, t_rest = 0;
    const int vm = choose_by_cost(tab, count, M, n_main, ksteps, block, cus, false, &ns, &t_main);
    if (vm < 0 || tab[vm].bm != 256 || tab[vm].bn != 256) return 0;
    const int vr = choose_by_cost(tab, count, M, N - n_main, ksteps, block, cus, false, &ns, &t_rest);
    if (vr < 0) return 0;
    if (t_split) *t_split = t_main + t_rest + 6.0;
    if (padding) *padding = padded_area(256, 256, M, n_main) + padded_area(tab[vr].bm, tab[vr].bn, M, N - n_main);
    if (g_ctx.row_split == 3 || whatever_the_estimate) return n_main;
    return t_main + t_rest + 6.0 < 0.975 * t_single ? n_main : 0;
}

int plan_nt(const NtProblem &q, Plan &pl, bool may_split_rows = true) {
    int count = 0;
    const Variant *tab = table_for(q.arith, q.block, q.kmaj, &count);
    if (!tab) return QGEMM_ERR_UNSUPPORTED;
    uint32_t model_split = 0;
    int vi = choose_variant(tab, count, q.M, q.N, ksteps_of(q), q.block, q.kmaj, g_ctx.num_cus, q.split_k == 0, &model_split);
    if (may_split_rows && vi >= 0 && !forced() && g_ctx.force_split <= 0 && q.split_k == 0 && model_split <= 1 &&
        q.M > 128 && q.kmaj == 0) {
        uint32_t ns = 0;
        double t_single = 0;
        const int ci = choose_by_cost(tab, count, q.M, q.N, ksteps_of(q), q.block, g_ctx.num_cus, false, &ns, &t_single);
        if (ci >= 0 && tab[ci].bm == tab[vi].bm && tab[ci].bn == tab[vi].bn && tab[ci].kgroups == tab[vi].kgroups) {
            double t_rows = 0, t_cols = 0;
            size_t pad_rows = 0, pad_cols = 0;
            size_t m_main = rows_for_full_rounds(tab, count, q.M, q.N, ksteps_of(q), q.block, g_ctx.num_cus, t_single, &t_rows, &pad_rows);
            size_t n_main = g_ctx.row_split == 2 ? 0
                                : cols_for_full_rounds(tab, count, q.M, q.N, ksteps_of(q), q.block, g_ctx.num_cus, t_single, &t_cols, &pad_cols, m_main != 0);
            // The columns by themselves where they are estimated at least 2.5 % ahead of the single launch, as the rows are.
            // Where the rows pass that test, the columns take their place if they are estimated 5 % faster, or no more
            // than 5 % slower with tiles that compute less beyond the matrix: the estimate prices tiles, not the rows in
            // them that count, and a full round of 256 tiles more than one of 252.  Config 4 is 14 row bands of 256 x 256
            // tiles and 2560 rows below on 192 x 256 ones, the last band of which is two thirds padding, or 10 column bands
            // and 2048 columns to the right that 32 x 8 such tiles cover exactly: 172.8 against 170.8 us, and 143.0
            // against 139.8 with per-matrix scales.  (Measured, the two are never further apart than 2.3 %.)
            if (g_ctx.row_split == 3) m_main = 0;
            if (m_main && n_main) {
                const bool cols = t_cols < 0.95 * t_rows || (t_cols <= 1.05 * t_rows && pad_cols < pad_rows);
                (cols ? m_main : n_main) = 0;
            }
            if (m_main || n_main) {
                NtProblem q_main = q, q_rest = q;
                if (m_main) {
                    q_main.M = m_main;
                    q_rest.M = q.M - m_main;
                } else {
                    q_main.N = n_main;
                    q_rest.N = q.N - n_main;
                }
                int st = plan_nt(q_main, pl, false);
                if (st != QGEMM_OK) return st;
                pl.rest.reset(new Plan());
                st = plan_nt(q_rest, *pl.rest, false);
                if (st != QGEMM_OK) return st;
                pl.m_main = m_main;
                pl.n_main = n_main;
                pl.split_bytes = std::max(pl.split_bytes, pl.rest->split_bytes);     // one after the other on the stream
                return QGEMM_OK;
            }
        }
    }
    if (forced()) {
        vi = row_by_name(tab, count, g_ctx.force_config);       // (a name this family does not have: unsupported)
        model_split = 0;
    }
    if (vi < 0) return QGEMM_ERR_UNSUPPORTED;
    const Variant &v = tab[vi];
    pl.v = &v;
    GemmArgs &a = pl.a;
    std::memset(&a, 0, sizeof(a));
    a.as = q.as;
    a.bs = q.bs;
    a.M = (uint32_t)q.M;
    a.N = (uint32_t)q.N;
    a.ksteps = (uint32_t)ksteps_of(q);
    a.k_tail = (uint32_t)(q.Kbytes % 128);
    a.lda = (uint32_t)q.lda_bytes;
    a.ldb = (uint32_t)q.ldb_bytes;
    a.tiles_m = (uint32_t)((q.M + v.bm - 1) / v.bm);
    a.tiles_n = (uint32_t)((q.N + v.bn - 1) / v.bn);
    a.group_m = g_ctx.force_group_m > 0 ? (uint32_t)g_ctx.force_group_m : 8;
    // Few rows (every workgroup streams a strip of B of its own out of memory, all of them at the same k): the workgroups
    // of column tile i (which share that strip of B and stay in step) start their K loops k_rot * i steps in and wrap
    // round, so that at any time the column tiles read at different offsets
    // inside their rows; with rows a power of two apart they otherwise all ask the same few memory channels
    // (16 x 28672 x 8192 fp8 with B out of HBM: 53 us from step 0, 45 - 46 us with 1, 2, 3 or 16 steps per workgroup,
    // 53 again with 32, i.e. 4 KiB; 8 steps are worse than none for the skinny-M kernel, whose waves share 16 steps).
    a.k_rot = g_ctx.k_rot >= 0 ? (uint32_t)g_ctx.k_rot : (q.M <= 256 ? 3u : 0u);
    a.as_ms = q.as_ms;
    a.as_ks = q.as_ks;
    a.bs_ns = q.bs_ns;
    a.bs_ks = q.bs_ks;
    a.nb_max = (uint32_t)((q.N + 127) / 128 - 1);
    // Copies of B with the streaming hint: where the launch reads B once (one row tile) and B is unlikely to be found in
    // the 256 MB memory-side cache by the next call (32 MiB or more: beyond what the L2s hold together).  With B out of
    // memory the hint is worth 2 - 12 %
    // (16 x 28672 x 8192 fp8 44.6 -> 40.2 us, 1 x 8192 x 8192 14.8 -> 13.0, 16 / 64 x 7168 x 2048 5.67 / 6.96 -> 5.40 / 6.75);
    // a caller who loops over one small B that sits in that cache loses 14 - 30 % with it (the same shapes with one B:
    // 3.56 / 5.04 -> 4.61 / 5.73), and with two row tiles sharing a strip of B it costs up to 8 %.  Option b_stream = 1
    // puts it on for every launch with one row tile: for callers whose weights do not stay in the cache between calls.
    a.b_stream = g_ctx.b_stream >= 0 ? (int)(g_ctx.b_stream && a.tiles_m == 1)
                                     : (a.tiles_m == 1 && q.N * q.Kbytes >= ((size_t)32 << 20));
    pl.tiles = (size_t)a.tiles_m * a.tiles_n;
    if (pl.tiles * 64 >= ((size_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;

    uint32_t nsplit = 1;
    if (q.split_k > 1) nsplit = (uint32_t)q.split_k;
    else if (q.split_k == 0) {
        if (g_ctx.force_split > 0) nsplit = (uint32_t)g_ctx.force_split;
        else if (model_split > 0) nsplit = model_split;
        else if (pl.tiles * 2 <= (size_t)g_ctx.num_cus && a.ksteps >= 8) {
            // enough slices to cover the CUs about twice, at least 4 K steps each
            uint32_t want = (uint32_t)((2 * (size_t)g_ctx.num_cus + pl.tiles - 1) / pl.tiles);
            nsplit = std::min<uint32_t>(want, a.ksteps / 4);
        }
    }
    nsplit = std::max<uint32_t>(1, std::min<uint32_t>(nsplit, a.ksteps));
    a.ksteps_per_split = (a.ksteps + nsplit - 1) / nsplit;
    nsplit = (a.ksteps + a.ksteps_per_split - 1) / a.ksteps_per_split;   // no empty slices
    a.nsplit = nsplit;
    pl.split_bytes = nsplit > 1 ? q.M * q.N * 4 * (size_t)nsplit : 0;
    return QGEMM_OK;
}

const char *kmaj_suffix(int kmaj) { return kmaj == 3 ? "_tn" : (kmaj == 2 ? "_nn" : ""); }

// split_ws: workspace of pl.split_bytes (ignored when the plan does not split)
int run_nt(const NtProblem &q, Plan &pl, void *split_ws, hipStream_t stream) {
    if (pl.rest) {
        // rows [0, m_main) with this plan, the rows below with the other: operands, scales and C move down m_main rows
        NtProblem q_main = q, q_rest = q;
        if (pl.m_main) {
            q_main.M = pl.m_main;
            q_rest.M = q.M - pl.m_main;
            q_rest.A = (const char *)q.A + pl.m_main * q.lda_bytes;            // (K-contiguous operands only: plan_nt)
            q_rest.C = (char *)q.C + pl.m_main * q.ldc * dtype_bytes(q.out_dtype);
            if (q.block && q.as) q_rest.as = q.as + pl.m_main * q.as_ms;
        } else {
            // columns [0, n_main) with this plan, the columns to the right with the other: B, its scale blocks and C move
            q_main.N = pl.n_main;
            q_rest.N = q.N - pl.n_main;
            q_rest.B = (const char *)q.B + pl.n_main * q.ldb_bytes;
            q_rest.C = (char *)q.C + pl.n_main * dtype_bytes(q.out_dtype);
            if (q.block && q.bs) q_rest.bs = q.bs + (pl.n_main / 128) * q.bs_ns;
        }
        std::unique_ptr<Plan> rest = std::move(pl.rest);
        int st = run_nt(q_main, pl, split_ws, stream);
        const std::string first = g_ctx.last_config;
        if (st == QGEMM_OK) st = run_nt(q_rest, *rest, split_ws, stream);
        g_ctx.last_config = first + (pl.m_main ? "+" : "|") + g_ctx.last_config;        // rows + rows below, columns | columns to the right
        pl.rest = std::move(rest);
        return st;
    }
    const Variant &v = *pl.v;
    GemmArgs &a = pl.a;
    a.A = (const char *)q.A;
    a.B = (const char *)q.B;
    a.as = q.as;
    a.bs = q.bs;
    a.as_ms = q.as_ms;
    a.as_ks = q.as_ks;
    a.bs_ns = q.bs_ns;
    a.bs_ks = q.bs_ks;
    a.as_groups = 0;
    if (q.block && v.kgroups == 2 && g_ctx.as_groups) {
        // K-contiguous a_scale on the rows with two K groups: four K blocks of a row per copy (GemmArgs::as_groups) where
        // rows and K slices start at multiples of four blocks; the rotated start then moves by four steps a column tile
        const bool slices4 = a.ksteps % 4 == 0 && (a.nsplit == 1 || a.ksteps_per_split % 4 == 0);
        const bool rows16 = q.as_ks == 1 && q.as_ms % 4 == 0 && ((uintptr_t)q.as & 15u) == 0;
        if (slices4 && rows16 && g_ctx.k_rot < 0 && a.k_rot) a.k_rot = 4;
        a.as_groups = slices4 && rows16 && a.k_rot % 4 == 0;
    }
#if QGEMM_DEBUG_BUILD
    a.dbg_cycles = (unsigned long long *)g_ctx.dbg_ptr;
#endif
    const bool i32_acc = q.arith == AR_I8 && !q.block;        // (int8 with block scales sums in fp32)
    if (a.nsplit == 1) {
        a.C = (char *)q.C;
        a.ldc = (uint32_t)q.ldc;
        a.out_dtype = q.out_dtype;
        a.per_matrix_scale = q.per_matrix;
        const int ob = dtype_bytes(q.out_dtype);
        const int vec = ob == 4 ? 16 : 8;
        a.vec_store = ((uintptr_t)q.C % vec == 0) && ((q.ldc * ob) % vec == 0);
        if (a.vec_store && (uintptr_t)q.C % 16 == 0 && (q.ldc * ob) % 16 == 0) a.vec_store = 2;
        // 4-byte C over at least three rounds of 256 x 256 tiles: spread the write bursts (see gemm_nt_kernel)
        // (with fewer than 32 K steps the offsets are too large a part of a tile's time: 7000 x 7168 x 2048 int8 to
        // f32 128 us without, 139 us with)
        const bool spread = v.bm == 256 && v.bn == 256 && ob == 4 && pl.tiles >= 3 * (size_t)g_ctx.num_cus && a.ksteps >= 32;
        a.stagger = g_ctx.stagger >= 0 ? (uint32_t)g_ctx.stagger : (spread ? 1u : 0u);
        // 4-byte C from 256 x 256 tiles: ordinary stores up to two rounds of tiles, non-temporal ones (and the staggered
        // start) from three on.  int8 to f32, ordinary against non-temporal, interleaved: 4096^3 59.1 against 61.1 us,
        // 4096 x 8192 x 4096 (two rounds) 114.2 against 124.0, 6144 x 8192 x 4096 (three) 165.6 against 169.9 with the
        // stagger, 8192^3 (four) 399.4 against 386.9; 2-byte C and every other tile are 1 - 6 % slower with ordinary
        // stores (the row with copying waves, 192 x 256, the K-group rows, 64 x 128).
        a.c_plain = g_ctx.c_plain >= 0 ? (int)g_ctx.c_plain
                                       : (v.bm == 256 && v.bn == 256 && ob == 4 && pl.tiles < 3 * (size_t)g_ctx.num_cus);
        a.stagger_wgs = (uint32_t)g_ctx.num_cus;
        a.stagger_groups = (uint32_t)std::max<long>(1, std::min<long>(32, g_ctx.stagger_groups));
        hipError_t e = v.launch(a, (uint32_t)pl.tiles, stream);
        g_ctx.last_config = std::string(v.name) + kmaj_suffix(q.kmaj);
        return e == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
    }

    // split-K: raw accumulators to the workspace, then one ordered reduction
    const size_t plane = q.M * q.N;
    a.C = (char *)split_ws;
    a.ldc = (uint32_t)q.N;
    a.split_stride = plane;
    a.out_dtype = i32_acc ? QGEMM_DT_I32 : QGEMM_DT_F32;
    a.per_matrix_scale = 0;
    a.vec_store = (q.N % 4 == 0) ? 2 : 0;   // workspace planes are 256-byte aligned, 4-byte elements
    hipError_t e = v.launch(a, (uint32_t)(pl.tiles * a.nsplit), stream);
    if (e != hipSuccess) return QGEMM_ERR_LAUNCH;

    ReduceArgs r;
    std::memset(&r, 0, sizeof(r));
    r.part = split_ws;
    r.C = q.C;
    r.as = q.as;
    r.bs = q.bs;
    r.M = (uint32_t)q.M;
    r.N = (uint32_t)q.N;
    r.nsplit = a.nsplit;
    r.ldc = q.ldc;
    r.plane = plane;
    r.part_is_i32 = i32_acc;
    r.out_dtype = q.out_dtype;
    r.per_matrix_scale = q.per_matrix;
    if (q.N % 4 == 0) {
        const int ob = dtype_bytes(q.out_dtype), c_align = ob == 4 ? 16 : 8;
        const int c_vec = (uintptr_t)q.C % c_align == 0 && (q.ldc * ob) % c_align == 0;
        const dim3 grid((unsigned)((plane / 4 + 255) / 256));
        if (i32_acc) hipLaunchKernelGGL(splitk_reduce4_kernel<true>, grid, dim3(256), 0, stream, r, c_vec);
        else hipLaunchKernelGGL(splitk_reduce4_kernel<false>, grid, dim3(256), 0, stream, r, c_vec);
    } else {
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((plane + 255) / 256)), dim3(256), 0, stream, r);
    }
    g_ctx.last_config = std::string(v.name) + kmaj_suffix(q.kmaj) + "_splitk" + std::to_string(a.nsplit);
    return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
}

// plan, get the split workspace (plus `extra` bytes behind it for transposed operands), run
int launch_transpose(int elem_bytes, const void *in, void *out, size_t M, size_t N, hipStream_t stream);

// The MFMA kernels read a_scale with the rows contiguous (a_scale[m + kb*M], the reference's own
// arrangement, hip_mix_gemm_kernel.cpp:149): 64 rows of one K block are one 256-byte request.  Scales
// given with K contiguous (a_scale[m*KB + kb]) are brought to that form first: M*KB floats, a few
// microseconds.  `room` is where in the workspace the copy goes.
// Which arrangement of a_scale the kernels of a block-scaled plan read.  Most want it rows-contiguous
// (a_scale[m + kb * ld], what QGEMM_LAYOUT_REFERENCE passes); the block-scaled 8-wave solo kernel has a twin
// (GemmCfg::ASK, table name "<name>_ks") that reads it with the K blocks contiguous, as QGEMM_LAYOUT_K_CONTIGUOUS
// passes it, two K blocks per 8-byte load (any number of K blocks per row and per K slice: see below).
// Puts the right one of each pair into the plan.  Returns true when the plan then reads q's scales as they are,
// false when they first have to be copied rows-contiguous (scales_rows_contiguous).
bool settle_scale_layout(const NtProblem &q, Plan &pl) {
    if (!q.block) return true;
    int count = 0;
    const Variant *tab = table_for(q.arith, q.block, q.kmaj, &count);
    auto partner = [&](const Variant *v, bool ks) -> const Variant * {      // the row of the pair with / without ASK
        if (v->a_scale_k_contiguous == ks) return v;
        return (tab && v->twin >= 0 && v->twin < count) ? &tab[v->twin] : nullptr;
    };
    if (q.as_ms == 1) {                                  // rows-contiguous: every kernel but the twins reads that
        for (Plan *p = &pl; p; p = p->rest.get())
            if (const Variant *v = partner(p->v, false)) p->v = v;
        return true;
    }
    // some other arrangement (K-contiguous, as QGEMM_LAYOUT_K_CONTIGUOUS passes it): fine where every launch of the
    // plan either takes any strides (simple pipeline, skinny-M kernel) or has a twin for it
    // (a twin fetches the scales of Variant::ks_blocks K blocks of a row per load, two or four: rows aligned to that
    // many floats, K and every K slice a multiple of that many blocks)
    bool as_is = true;
    for (const Plan *p = &pl; as_is && p; p = p->rest.get()) {
        if (p->v->a_scale_any_stride) continue;
        const Variant *twin = partner(p->v, true);
        if (!twin || q.as_ks != 1) {
            as_is = false;
            break;
        }
        const uint32_t g = (uint32_t)twin->ks_blocks;
        // (two K blocks per load, into registers: any row length and any slice.  An 8-byte buffer load needs 4-byte
        // alignment only, the pair that starts with a row's last block ends with the next row's first, which nobody
        // uses, and at the end of the array the range check, which is per dword, returns zero for it: probed by
        // qgemm_selftest_layouts.  Four blocks per copy go through LDS and keep their alignment rules.)
        as_is = g == 2 ? ((uintptr_t)q.as % 4) == 0
                       : (g > 0 && q.as_ms % g == 0 && ((uintptr_t)q.as % (4 * g)) == 0 && p->a.ksteps % g == 0 &&
                          !(p->a.nsplit > 1 && p->a.ksteps_per_split % g != 0));
    }
    for (Plan *p = &pl; p; p = p->rest.get()) {
        if (p->v->a_scale_any_stride) continue;
        if (const Variant *v = partner(p->v, as_is)) p->v = v;
    }
    return as_is;
}

int scales_rows_contiguous(NtProblem &q, void *room, hipStream_t stream) {
    if (!q.block || q.as_ms == 1) return QGEMM_OK;
    const size_t KB = (q.Kbytes + 127) / 128;
    int st = launch_transpose(4, q.as, room, q.M, KB, stream);
    if (st != QGEMM_OK) return st;
    q.as = (const float *)room;
    q.as_ms = 1;
    q.as_ks = (uint32_t)q.M;
    return QGEMM_OK;
}
size_t scales_room(const NtProblem &q) {
    if (!q.block || q.as_ms == 1) return 0;
    return (q.M * ((q.Kbytes + 127) / 128) * 4 + 255) / 256 * 256;
}

int launch_nt(NtProblem q, hipStream_t stream) {
    Plan pl;
    int st = plan_nt(q, pl);
    if (st != QGEMM_OK) return st;
    void *ws = nullptr;
    const size_t split_room = (pl.split_bytes + 255) / 256 * 256;
    const size_t as_room = settle_scale_layout(q, pl) ? 0 : scales_room(q);
    if (split_room + as_room) {
        st = ensure_workspace_locked(split_room + as_room, stream, &ws);
        if (st != QGEMM_OK) return st;
    }
    if (as_room) {
        st = scales_rows_contiguous(q, (char *)ws + split_room, stream);      // (run_nt takes the scales from q)
        if (st != QGEMM_OK) return st;
    }
    return run_nt(q, pl, ws, stream);
}

template <int DT>
int launch_strided_t(const StridedArgs &s, hipStream_t stream) {
    dim3 grid((s.N + 15) / 16, (s.M + 15) / 16);
    hipLaunchKernelGGL(gemm_strided_kernel<DT>, grid, dim3(256), 0, stream, s);
    return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
}

int launch_strided(int in_dtype, const StridedArgs &s, hipStream_t stream) {
    g_ctx.last_config = "strided_any_shape";
    if ((s.N + 15) / 16 > 0x7FFFFFFFu || (s.M + 15) / 16 > 65535u) return QGEMM_ERR_TOO_LARGE;    // grid limits
    switch (in_dtype) {
        case QGEMM_DT_I8: return launch_strided_t<QGEMM_DT_I8>(s, stream);
        case QGEMM_DT_F8E4M3: return launch_strided_t<QGEMM_DT_F8E4M3>(s, stream);
        case QGEMM_DT_BF16: return launch_strided_t<QGEMM_DT_BF16>(s, stream);
        case QGEMM_DT_F16: return launch_strided_t<QGEMM_DT_F16>(s, stream);
    }
    return QGEMM_ERR_UNSUPPORTED;
}

int launch_transpose(int elem_bytes, const void *in, void *out, size_t M, size_t N, hipStream_t stream) {
    if (M == 0 || N == 0) return QGEMM_OK;
    if (M >= ((size_t)1 << 31) || N >= ((size_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
    if (grid.y > 65535u * 1024u) return QGEMM_ERR_TOO_LARGE;
    if (elem_bytes == 1 && M % 16 == 0 && N % 4 == 0 && (uintptr_t)in % 4 == 0 && (uintptr_t)out % 16 == 0) {
        dim3 g128((unsigned)((N + 127) / 128), (unsigned)((M + 127) / 128));
        hipLaunchKernelGGL(transpose_bytes_kernel, g128, dim3(256), 0, stream, (const uint8_t *)in, (uint8_t *)out,
                           (uint32_t)M, (uint32_t)N);
        return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
    }
    if (elem_bytes == 2 && M % 8 == 0 && N % 8 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
        dim3 g((unsigned)((N + 255) / 256), (unsigned)((M + 63) / 64));
        hipLaunchKernelGGL(transpose_u16_kernel, g, dim3(256), 0, stream, (const uint16_t *)in, (uint16_t *)out,
                           (uint32_t)M, (uint32_t)N);
        return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
    }
    switch (elem_bytes) {
        case 1:
            hipLaunchKernelGGL(transpose_kernel<uint8_t>, grid, dim3(256), 0, stream, (const uint8_t *)in, (uint8_t *)out,
                               (uint32_t)M, (uint32_t)N);
            break;
        case 2:
            hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, stream, (const uint16_t *)in,
                               (uint16_t *)out, (uint32_t)M, (uint32_t)N);
            break;
        case 4:
            hipLaunchKernelGGL(transpose_kernel<uint32_t>, grid, dim3(256), 0, stream, (const uint32_t *)in,
                               (uint32_t *)out, (uint32_t)M, (uint32_t)N);
            break;
        default: return QGEMM_ERR_UNSUPPORTED;
    }
    return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
}

template <int IN_DT>
int quantize_t(int mode, QuantArgs &a, hipStream_t stream) {
    const uint64_t groups = (uint64_t)a.rows * ((a.cols + 3) / 4);
    if (mode == QGEMM_QUANT_PER_MATRIX) {
        // two passes: partial maxima (one per workgroup) into the workspace, then scale and cast
        const uint32_t nblk = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>(2048, (groups + 1023) / 1024));
        void *ws = nullptr;
        int st = ensure_workspace_locked(nblk * sizeof(float), stream, &ws);
        if (st != QGEMM_OK) return st;
        a.partial = (float *)ws;
        a.npartial = nblk;
        hipLaunchKernelGGL(quant_amax_kernel<IN_DT>, dim3(nblk), dim3(256), 0, stream, a);
        const uint32_t nq = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>(8192, (groups + 255) / 256));
        hipLaunchKernelGGL(quant_matrix_kernel<IN_DT>, dim3(nq), dim3(256), 0, stream, a);
    } else if (mode == QGEMM_QUANT_BLOCK_1x128) {
        const uint64_t nblocks = (uint64_t)a.rows * ((a.cols + 127) / 128);
        if ((nblocks + 7) / 8 >= ((uint64_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
        const uint32_t nbc = a.cols / 128;
        const bool whole = a.cols % 128 == 0 && a.ld % 4 == 0 && (uintptr_t)a.x % 16 == 0 && a.ldq % 4 == 0 &&
                           (uintptr_t)a.q % 4 == 0 && a.out_dtype == QGEMM_DT_F8E4M3 && (nbc + 7) / 8 <= 65535 && a.rows > 0;
        if (whole)
            hipLaunchKernelGGL(quant_row_block_whole_kernel<IN_DT>, dim3(a.rows, (nbc + 7) / 8), dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL(quant_row_block_kernel<IN_DT>, dim3((unsigned)((nblocks + 7) / 8)), dim3(256), 0, stream, a);
    } else {
        const uint64_t nblocks = (uint64_t)((a.rows + 127) / 128) * ((a.cols + 127) / 128);
        if (nblocks >= ((uint64_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
        const bool whole = a.cols % 128 == 0 && a.rows % 128 == 0 && a.rows > 0 && a.cols > 0 && a.ld % 4 == 0 &&
                           (uintptr_t)a.x % 16 == 0 && a.ldq % 4 == 0 && (uintptr_t)a.q % 4 == 0 &&
                           a.out_dtype == QGEMM_DT_F8E4M3 && a.rows / 128 <= 65535;
        if (whole)
            hipLaunchKernelGGL(quant_square_block_whole_kernel<IN_DT>, dim3(a.cols / 128, a.rows / 128), dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL(quant_square_block_kernel<IN_DT>, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
    }
    return hipGetLastError() == hipSuccess ? QGEMM_OK : QGEMM_ERR_LAUNCH;
}

}  // namespace

// ===========================================================================
extern "C" {

QGEMM_EXPORT int qgemm_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

QGEMM_EXPORT int qgemm_init(void) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    return ensure_init_locked();
}

QGEMM_EXPORT int qgemm_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (g_ctx.ws.p || !g_ctx.retired.empty()) {
        (void)hipDeviceSynchronize();
        if (g_ctx.ws.p) (void)hipFree(g_ctx.ws.p);
        for (void *p : g_ctx.retired) (void)hipFree(p);
    }
    if (g_ctx.ws_event) (void)hipEventDestroy(g_ctx.ws_event);
    g_ctx.ws = WsBlock();
    g_ctx.retired.clear();
    g_ctx.ws_event = nullptr;
    g_ctx.ws_event_recorded = false;
    g_ctx.ready = false;
    return QGEMM_OK;
}

QGEMM_EXPORT const char *qgemm_status_string(int status) {
    switch (status) {
        case QGEMM_OK: return "ok";
        case QGEMM_ERR_INVALID_ARG: return "invalid argument";
        case QGEMM_ERR_UNSUPPORTED: return "unsupported dtype / layout combination";
        case QGEMM_ERR_NO_DEVICE: return "no HIP device";
        case QGEMM_ERR_LAUNCH: return "HIP call failed";
        case QGEMM_ERR_ALLOC: return "workspace allocation failed";
        case QGEMM_ERR_NOT_DIVISIBLE_M: return "M is not divisible by any predefined BLOCK_TILE_SIZE_M in the list";
        case QGEMM_ERR_NOT_DIVISIBLE_N: return "N is not divisible by any predefined BLOCK_TILE_SIZE_N in the list";
        case QGEMM_ERR_NOT_DIVISIBLE_K: return "K is not divisible by any predefined BLOCK_TILE_SIZE_K in the list";
        case QGEMM_ERR_TOO_LARGE: return "dimension or stride too large";
        case QGEMM_ERR_SCRATCH_TOO_SMALL: return "problem needs more than the static scratch (QGEMM_STATIC_SCRATCH_BYTES)";
    }
    return "unknown status";
}

QGEMM_EXPORT int qgemm_tile_map(uint32_t wg, uint32_t tiles_m, uint32_t tiles_n, uint32_t group_m, uint32_t *tile_m,
                   uint32_t *tile_n) {
    if (!tile_m || !tile_n || tiles_m == 0 || tiles_n == 0) return QGEMM_ERR_INVALID_ARG;
    if ((uint64_t)wg >= (uint64_t)tiles_m * tiles_n) return QGEMM_ERR_INVALID_ARG;
    tile_map(wg, tiles_m, tiles_n, group_m, *tile_m, *tile_n);
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_set_option(const char *key, long value) {
    if (!key) return QGEMM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (!std::strcmp(key, "force_config")) {
        if (value != -1) return QGEMM_ERR_INVALID_ARG;      // rows are named: qgemm_force_config; -1 returns to the heuristic
        g_ctx.force_config.clear();
    } else if (!std::strcmp(key, "force_split")) g_ctx.force_split = value;
    else if (!std::strcmp(key, "group_m")) g_ctx.force_group_m = value;
    else if (!std::strcmp(key, "kmajor")) g_ctx.kmajor = value;
    else if (!std::strcmp(key, "stagger")) g_ctx.stagger = value;
    else if (!std::strcmp(key, "stagger_groups")) g_ctx.stagger_groups = value;
    else if (!std::strcmp(key, "c_plain")) g_ctx.c_plain = value;
    else if (!std::strcmp(key, "b_stream")) g_ctx.b_stream = value;
    else if (!std::strcmp(key, "k_rot")) g_ctx.k_rot = value;
    else if (!std::strcmp(key, "as_groups")) g_ctx.as_groups = value;
    else if (!std::strcmp(key, "small_tiles")) g_ctx.small_tiles = value;
#if QGEMM_DEBUG_BUILD
    else if (!std::strcmp(key, "dbg_ptr")) g_ctx.dbg_ptr = value;
#endif
    else if (!std::strcmp(key, "row_split")) g_ctx.row_split = value;
    else return QGEMM_ERR_INVALID_ARG;
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_force_config(const char *name) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (!name || !*name) {
        g_ctx.force_config.clear();
        return QGEMM_OK;
    }
    // the name has to be a row of at least one family
    bool known = false;
    for (int arith = 0; arith < 4 && !known; ++arith)
        for (int block = 0; block < 2 && !known; ++block)
            for (int kmaj = 0; kmaj < 4 && !known; ++kmaj) {
                int count = 0;
                const Variant *tab = table_for(arith, block != 0, kmaj, &count);
                known = row_by_name(tab, count, name) >= 0;
            }
    if (!known) return QGEMM_ERR_INVALID_ARG;
    g_ctx.force_config = name;
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_variant_count(int in_dtype, int scale_mode, int k_major) {
    int count = 0;
    const int arith = arith_of(in_dtype);
    if (arith < 0 || !table_for(arith, scale_mode == QGEMM_SCALE_BLOCK128, k_major, &count)) return 0;
    return count;
}

QGEMM_EXPORT int qgemm_variant_name(int in_dtype, int scale_mode, int k_major, int index, char *buf, size_t buflen) {
    if (!buf || buflen == 0) return QGEMM_ERR_INVALID_ARG;
    int count = 0;
    const int arith = arith_of(in_dtype);
    const Variant *tab = arith < 0 ? nullptr : table_for(arith, scale_mode == QGEMM_SCALE_BLOCK128, k_major, &count);
    if (!tab) return QGEMM_ERR_UNSUPPORTED;
    if (index < 0 || index >= count) return QGEMM_ERR_INVALID_ARG;
    std::snprintf(buf, buflen, "%s", tab[index].name);
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_last_config(char *buf, size_t buflen) {
    if (!buf || buflen == 0) return QGEMM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    std::snprintf(buf, buflen, "%s", g_ctx.last_config.c_str());
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_plan(int in_dtype, int scale_mode, int k_major, size_t M, size_t N, size_t K, char *buf,
                            size_t buflen) {
    if (!buf || buflen == 0 || M == 0 || N == 0 || K == 0 || k_major < 0 || k_major > 3) return QGEMM_ERR_INVALID_ARG;
    const int arith = arith_of(in_dtype);
    if (arith < 0) return QGEMM_ERR_UNSUPPORTED;
    if (scale_mode != 0 && scale_mode != QGEMM_SCALE_PER_MATRIX && scale_mode != QGEMM_SCALE_BLOCK128)
        return QGEMM_ERR_INVALID_ARG;
    if (scale_mode == QGEMM_SCALE_BLOCK128 && arith != AR_F8 && arith != AR_I8) return QGEMM_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_ctx.mu);          // no device call below: 256 CUs are assumed before qgemm_init
    const size_t eb = (arith == AR_BF16 || arith == AR_F16) ? 2 : 1;
    NtProblem q;
    std::memset(&q, 0, sizeof(q));
    q.arith = arith;
    q.block = scale_mode == QGEMM_SCALE_BLOCK128;
    q.M = M;
    q.N = N;
    q.Kbytes = K * eb;
    q.lda_bytes = q.ldb_bytes = K * eb;
    q.ldc = N;
    std::string name;
    if (k_major) {
        const size_t lda = (k_major & 1) ? M * eb : K * eb, ldb = (k_major & 2) ? N * eb : K * eb;
        int rows = 0;
        const bool family = table_for(arith, q.block, k_major, &rows) != nullptr;
        if (family && kmajor_problem_ok(q, k_major, lda, ldb)) {
            q.kmaj = k_major;
            q.lda_bytes = lda;
            q.ldb_bytes = ldb;
        } else {
            name = "transpose+";
        }
    }
    if (!mfma_shape_ok(q)) {
        std::snprintf(buf, buflen, "strided_any_shape");
        return QGEMM_OK;
    }
    Plan pl;
    const int st = plan_nt(q, pl);
    if (st != QGEMM_OK) return st;
    if (q.block) {          // dense scales in the arrangement of the layout asked about
        const uint32_t KB = (uint32_t)((K + 127) / 128);
        if (k_major == 3) { q.as_ms = 1; q.as_ks = (uint32_t)M; }
        else { q.as_ms = KB; q.as_ks = 1; }
        (void)settle_scale_layout(q, pl);
    }
    name += std::string(pl.v->name) + kmaj_suffix(q.kmaj);
    if (pl.a.nsplit > 1) name += "_splitk" + std::to_string(pl.a.nsplit);
    if (pl.rest) {
        name += (pl.m_main ? "+" : "|") + std::string(pl.rest->v->name);
        if (pl.rest->a.nsplit > 1) name += "_splitk" + std::to_string(pl.rest->a.nsplit);
    }
    std::snprintf(buf, buflen, "%s", name.c_str());
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_quantize(int in_dtype, int out_dtype, int mode, const void *x, size_t ld, size_t rows, size_t cols,
                                void *q, size_t ldq, float *scales, size_t scale_rs, size_t scale_cs, void *stream_) {
    if (in_dtype != QGEMM_DT_F32 && in_dtype != QGEMM_DT_BF16 && in_dtype != QGEMM_DT_F16) return QGEMM_ERR_UNSUPPORTED;
    if (out_dtype != QGEMM_DT_I8 && out_dtype != QGEMM_DT_F8E4M3) return QGEMM_ERR_UNSUPPORTED;
    if (mode != QGEMM_QUANT_PER_MATRIX && mode != QGEMM_QUANT_BLOCK_1x128 && mode != QGEMM_QUANT_BLOCK_128x128)
        return QGEMM_ERR_INVALID_ARG;
    if (!scales) return QGEMM_ERR_INVALID_ARG;
    if (rows >= ((size_t)1 << 31) || cols >= ((size_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    hipStream_t stream = (hipStream_t)stream_;
    WorkspaceUse ws_use(stream);
    QuantArgs a;
    std::memset(&a, 0, sizeof(a));
    a.x = x;
    a.q = q;
    a.scales = scales;
    a.rows = (uint32_t)rows;
    a.cols = (uint32_t)cols;
    a.ld = ld;
    a.ldq = ldq;
    a.scale_rs = scale_rs;
    a.scale_cs = scale_cs;
    a.out_dtype = out_dtype;
    if (rows == 0 || cols == 0) {
        if (mode != QGEMM_QUANT_PER_MATRIX) return QGEMM_OK;
        // the scale of an empty matrix is the scale of a zero matrix: run the passes over nothing
        a.rows = a.cols = 0;
    } else if (!x || !q || ld < cols || ldq < cols) {
        return QGEMM_ERR_INVALID_ARG;
    }
    g_ctx.last_config = mode == QGEMM_QUANT_PER_MATRIX ? "quantize_per_matrix"
                        : (mode == QGEMM_QUANT_BLOCK_1x128 ? "quantize_1x128" : "quantize_128x128");
    switch (in_dtype) {
        case QGEMM_DT_F32: return quantize_t<QGEMM_DT_F32>(mode, a, stream);
        case QGEMM_DT_BF16: return quantize_t<QGEMM_DT_BF16>(mode, a, stream);
        default: return quantize_t<QGEMM_DT_F16>(mode, a, stream);
    }
}

QGEMM_EXPORT int qgemm_transpose(int elem_bytes, const void *in, void *out, size_t M, size_t N, void *stream) {
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) return QGEMM_ERR_UNSUPPORTED;
    if (M == 0 || N == 0) return QGEMM_OK;
    if (!in || !out) return QGEMM_ERR_INVALID_ARG;
    if (M >= ((size_t)1 << 31) || N >= ((size_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    return launch_transpose(elem_bytes, in, out, M, N, (hipStream_t)stream);
}

QGEMM_EXPORT int qgemm_gemm(int in_dtype, int out_dtype, int layout_b, const void *A, size_t ldA, const void *B, size_t ldB,
               void *C, size_t ldC, size_t M, size_t N, size_t K, void *stream_) {
    const int arith = arith_of(in_dtype);
    if (arith < 0 || !out_dtype_ok(in_dtype, out_dtype)) return QGEMM_ERR_UNSUPPORTED;
    if (layout_b != QGEMM_B_KN && layout_b != QGEMM_B_NK) return QGEMM_ERR_INVALID_ARG;
    if (M == 0 || N == 0) return QGEMM_OK;
    if (!A || !B || !C || K == 0) return QGEMM_ERR_INVALID_ARG;
    if (ldA < K || ldC < N || ldB < (layout_b == QGEMM_B_KN ? N : K)) return QGEMM_ERR_INVALID_ARG;
    hipStream_t stream = (hipStream_t)stream_;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    WorkspaceUse ws_use(stream);

    const size_t eb = dtype_bytes(in_dtype);
    NtProblem q;
    std::memset(&q, 0, sizeof(q));
    q.arith = arith;
    q.block = false;
    q.A = A;
    q.C = C;
    q.lda_bytes = ldA * eb;
    q.ldc = ldC;
    q.M = M;
    q.N = N;
    q.Kbytes = K * eb;
    q.out_dtype = out_dtype;
    q.per_matrix = 0;
    q.split_k = 0;

    if (layout_b == QGEMM_B_NK) {
        q.B = B;
        q.ldb_bytes = ldB * eb;
        if (mfma_shape_ok(q) && aligned16(A) && aligned16(B)) return launch_nt(q, stream);
    } else if (eb == 2 && aligned16(A) && aligned16(B) && kmajor_problem_ok(q, 2, q.lda_bytes, ldB * eb)) {
        // "NN", 16-bit operands: the kernel takes B as it is stored (K x N), see GemmCfg::KMAJ
        q.kmaj = 2;
        q.B = B;
        q.ldb_bytes = ldB * eb;
        return launch_nt(q, stream);
    } else if (ldB == N) {
        // "NN" otherwise: bring B to N x K through the transpose utility (the route the reference's
        // v3.1 launcher sketches, sm80_gemm_kernel_v3.1.cu:277-279), then run the NT kernel.
        q.ldb_bytes = K * eb;
        if (mfma_shape_ok(q) && aligned16(A)) {
            Plan pl;
            st = plan_nt(q, pl);
            if (st != QGEMM_OK) return st;
            const size_t split_room = (pl.split_bytes + 255) / 256 * 256;
            void *ws = nullptr;
            st = ensure_workspace_locked(split_room + N * K * eb, stream, &ws);
            if (st != QGEMM_OK) return st;
            void *bt = (char *)ws + split_room;
            st = launch_transpose((int)eb, B, bt, K, N, stream);
            if (st != QGEMM_OK) return st;
            q.B = bt;
            return run_nt(q, pl, ws, stream);
        }
    }

    if (M >= ((size_t)1 << 32) || N >= ((size_t)1 << 32) || K >= ((size_t)1 << 32)) return QGEMM_ERR_TOO_LARGE;
    StridedArgs s;
    std::memset(&s, 0, sizeof(s));
    s.A = A;
    s.B = B;
    s.C = C;
    s.M = (uint32_t)M;
    s.N = (uint32_t)N;
    s.K = (uint32_t)K;
    s.a_rs = ldA;
    s.a_cs = 1;
    if (layout_b == QGEMM_B_NK) {
        s.b_ns = ldB;
        s.b_ks = 1;
    } else {
        s.b_ns = 1;
        s.b_ks = ldB;
    }
    s.ldc = ldC;
    s.out_dtype = out_dtype;
    s.scale_mode = 0;
    return launch_strided(in_dtype, s, stream);
}

}  // extern "C"

namespace {

// Body of qgemm_scaled_gemm and qgemm_scaled_gemm_static; `use_static`: the workspace is the static scratch.
int scaled_gemm_entry(bool use_static, int in_dtype, int out_dtype, int scale_mode, int layout, const void *A, const void *B,
                      const float *a_scale, const float *b_scale, void *C, size_t ldC, size_t M, size_t N, size_t K,
                      int split_k, void *stream_) {
    if (in_dtype != QGEMM_DT_I8 && in_dtype != QGEMM_DT_F8E4M3) return QGEMM_ERR_UNSUPPORTED;
    if (!out_dtype_ok(in_dtype, out_dtype)) return QGEMM_ERR_UNSUPPORTED;
    if (scale_mode != QGEMM_SCALE_PER_MATRIX && scale_mode != QGEMM_SCALE_BLOCK128) return QGEMM_ERR_INVALID_ARG;
    // (int8 with block scales and int32 output: there is no int32 sum of scaled blocks)
    if (scale_mode == QGEMM_SCALE_BLOCK128 && out_dtype == QGEMM_DT_I32) return QGEMM_ERR_UNSUPPORTED;
    if (layout != QGEMM_LAYOUT_K_CONTIGUOUS && layout != QGEMM_LAYOUT_REFERENCE) return QGEMM_ERR_INVALID_ARG;
    if (split_k < 0) return QGEMM_ERR_INVALID_ARG;
    if (layout == QGEMM_LAYOUT_REFERENCE) {
        // dispatch contract of select_BLOCK_TILE_SIZE_{M,N,K}: hip_mix_gemm_kernel.cpp:442-505
        if (M % 32 != 0) return QGEMM_ERR_NOT_DIVISIBLE_M;
        if (N % 32 != 0) return QGEMM_ERR_NOT_DIVISIBLE_N;
        if (K % 32 != 0) return QGEMM_ERR_NOT_DIVISIBLE_K;
    }
    if (M == 0 || N == 0) return QGEMM_OK;
    if (!A || !B || !C || K == 0 || ldC < N) return QGEMM_ERR_INVALID_ARG;
    const bool raw_acc = out_dtype == QGEMM_DT_I32;
    if (!raw_acc && (!a_scale || !b_scale)) return QGEMM_ERR_INVALID_ARG;
    hipStream_t stream = (hipStream_t)stream_;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    struct StaticScope {        // every workspace request of this call goes to the static scratch
        explicit StaticScope(bool on) { g_ctx.static_call = on; }
        ~StaticScope() { g_ctx.static_call = false; }
    } scope(use_static);
    WorkspaceUse ws_use(stream);

    const bool block = scale_mode == QGEMM_SCALE_BLOCK128;
    const uint32_t KB = (uint32_t)((K + 127) / 128), NBLK = (uint32_t)((N + 127) / 128);
    NtProblem q;
    std::memset(&q, 0, sizeof(q));
    q.arith = arith_of(in_dtype);
    q.block = block;
    q.C = C;
    q.ldc = ldC;
    q.M = M;
    q.N = N;
    q.Kbytes = K;
    q.lda_bytes = K;
    q.ldb_bytes = K;
    q.as = a_scale;
    q.bs = b_scale;
    q.out_dtype = out_dtype;
    q.per_matrix = (!block && !raw_acc) ? 1 : 0;
    q.split_k = split_k;
    if (block) {
        if (layout == QGEMM_LAYOUT_K_CONTIGUOUS) {
            q.as_ms = KB; q.as_ks = 1; q.bs_ns = KB; q.bs_ks = 1;
        } else {   // a_scale[m + kb*M], b_scale[nb + kb*ceil(N/128)]: hip_mix_gemm_kernel.cpp:137,149,164
            q.as_ms = 1; q.as_ks = (uint32_t)M; q.bs_ns = 1; q.bs_ks = NBLK;
        }
    }

    if (layout == QGEMM_LAYOUT_K_CONTIGUOUS) {
        q.A = A;
        q.B = B;
        if (mfma_shape_ok(q) && aligned16(A) && aligned16(B)) return launch_nt(q, stream);
    } else if (block && aligned16(A) && aligned16(B) && kmajor_problem_ok(q, 3, M, N)) {
        // reference layout, block scales: A is K x M (M contiguous), B is K x N; the kernel reads both as stored
        q.kmaj = 3;
        q.A = A;
        q.B = B;
        q.lda_bytes = M;
        q.ldb_bytes = N;
        return launch_nt(q, stream);
    } else if (mfma_shape_ok(q)) {
        // reference layout otherwise: bring both to K-contiguous through the transpose utility, then run
        // the NT kernel.
        Plan pl;
        st = plan_nt(q, pl);
        if (st != QGEMM_OK) return st;
        const size_t split_room = (pl.split_bytes + 255) / 256 * 256;
        const size_t at_bytes = (M * K + 255) / 256 * 256;
        void *ws = nullptr;
        st = ensure_workspace_locked(split_room + at_bytes + N * K, stream, &ws);
        if (st != QGEMM_OK) return st;
        char *at = (char *)ws + split_room, *bt = at + at_bytes;
        // M, N, K are multiples of 32 here: both matrices qualify for the register-permute byte transpose
        if (aligned16(A) && aligned16(B) && K < ((size_t)1 << 31)) {
            Transpose2Args t;
            t.in[0] = (const uint8_t *)A; t.out[0] = (uint8_t *)at; t.M[0] = (uint32_t)K; t.N[0] = (uint32_t)M;
            t.in[1] = (const uint8_t *)B; t.out[1] = (uint8_t *)bt; t.M[1] = (uint32_t)K; t.N[1] = (uint32_t)N;
            const size_t tk = (K + 127) / 128;
            t.tiles_n[0] = (uint32_t)((M + 127) / 128);
            t.tiles_n[1] = (uint32_t)((N + 127) / 128);
            t.tiles0 = (uint32_t)(tk * t.tiles_n[0]);
            const size_t total = tk * ((size_t)t.tiles_n[0] + t.tiles_n[1]);
            if (total >= ((size_t)1 << 31)) return QGEMM_ERR_TOO_LARGE;
            hipLaunchKernelGGL(transpose_bytes2_kernel, dim3((unsigned)total), dim3(256), 0, stream, t);
            if (hipGetLastError() != hipSuccess) return QGEMM_ERR_LAUNCH;
        } else {
            st = launch_transpose(1, A, at, K, M, stream);
            if (st != QGEMM_OK) return st;
            st = launch_transpose(1, B, bt, K, N, stream);
            if (st != QGEMM_OK) return st;
        }
        q.A = at;
        q.B = bt;
        (void)settle_scale_layout(q, pl);            // (scales are rows-contiguous in this layout)
        return run_nt(q, pl, ws, stream);
    }

    if (M >= ((size_t)1 << 32) || N >= ((size_t)1 << 32) || K >= ((size_t)1 << 32)) return QGEMM_ERR_TOO_LARGE;
    StridedArgs s;
    std::memset(&s, 0, sizeof(s));
    s.A = A;
    s.B = B;
    s.C = C;
    s.as = a_scale;
    s.bs = b_scale;
    s.M = (uint32_t)M;
    s.N = (uint32_t)N;
    s.K = (uint32_t)K;
    if (layout == QGEMM_LAYOUT_K_CONTIGUOUS) {
        s.a_rs = K; s.a_cs = 1; s.b_ns = K; s.b_ks = 1;
    } else {
        s.a_rs = 1; s.a_cs = M; s.b_ns = 1; s.b_ks = N;
    }
    s.ldc = ldC;
    s.as_ms = q.as_ms; s.as_ks = q.as_ks; s.bs_ns = q.bs_ns; s.bs_ks = q.bs_ks;
    // partial products per reference K tile: first of {128, 64, 32} dividing K (:442-463)
    s.bk = K % 128 == 0 ? 128 : (K % 64 == 0 ? 64 : (K % 32 == 0 ? 32 : 128));
    s.out_dtype = out_dtype;
    s.scale_mode = raw_acc ? 0 : scale_mode;
    return launch_strided(in_dtype, s, stream);
}

}  // namespace

extern "C" {

QGEMM_EXPORT int qgemm_scaled_gemm(int in_dtype, int out_dtype, int scale_mode, int layout, const void *A, const void *B,
                      const float *a_scale, const float *b_scale, void *C, size_t ldC, size_t M, size_t N, size_t K,
                      int split_k, void *stream) {
    return scaled_gemm_entry(false, in_dtype, out_dtype, scale_mode, layout, A, B, a_scale, b_scale, C, ldC, M, N, K, split_k,
                             stream);
}

QGEMM_EXPORT int qgemm_scaled_gemm_static(int in_dtype, int out_dtype, int scale_mode, int layout, const void *A,
                                          const void *B, const float *a_scale, const float *b_scale, void *C, size_t ldC,
                                          size_t M, size_t N, size_t K, int split_k, void *stream) {
    return scaled_gemm_entry(true, in_dtype, out_dtype, scale_mode, layout, A, B, a_scale, b_scale, C, ldC, M, N, K, split_k,
                             stream);
}

QGEMM_EXPORT int qgemm_reserve_workspace(size_t bytes) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    if (bytes <= g_ctx.ws.bytes) return QGEMM_OK;
    // (takes no stream, so it cannot tell whether one is being captured: the caller reserves before a capture)
    // grow geometrically, as ensure_workspace_locked does: a caller that reserves step by step then retires
    // O(log n) blocks, not one per call
    const size_t want = std::max(bytes, 2 * g_ctx.ws.bytes);
    void *p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) {
        (void)hipGetLastError();
        return QGEMM_ERR_ALLOC;
    }
    if (g_ctx.ws.p) g_ctx.retired.push_back(g_ctx.ws.p);
    g_ctx.ws.p = p;
    g_ctx.ws.bytes = want;
    return QGEMM_OK;
}

QGEMM_EXPORT int qgemm_workspace_info(void **base, size_t *bytes) {
    if (!base || !bytes) return QGEMM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    *base = g_ctx.ws.p;
    *bytes = g_ctx.ws.bytes;
    return QGEMM_OK;
}

// ---------------------------------------------------------------------------
// self test
// ---------------------------------------------------------------------------
namespace {

float host_decode(int arith, const uint8_t *p, int idx) {
    if (arith == AR_I8) return (float)((const int8_t *)p)[idx];
    if (arith == AR_F8) {
        const uint8_t b = p[idx];
        const int e = (b >> 3) & 15, m = b & 7;
        float mag = e == 0 ? (float)m / 512.0f : (1.0f + (float)m / 8.0f) * std::exp2((float)(e - 7));
        return (b & 0x80) ? -mag : mag;
    }
    uint16_t h;
    std::memcpy(&h, p + 2 * idx, 2);
    if (arith == AR_BF16) {
        uint32_t u = (uint32_t)h << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
    // fp16: the probe only uses small integers, exactly representable
    const int e = (h >> 10) & 31, m = h & 1023;
    float mag = e == 0 ? (float)m / 16777216.0f : (1.0f + (float)m / 1024.0f) * std::exp2((float)(e - 15));
    return (h & 0x8000) ? -mag : mag;
}

// value v in [-4, 4] encoded in the family's element type
void host_encode_small(int arith, int v, uint8_t *p, int idx) {
    if (arith == AR_I8) { ((int8_t *)p)[idx] = (int8_t)v; return; }
    if (arith == AR_F8) {
        static const uint8_t code[5] = {0x00, 0x38, 0x40, 0x44, 0x48};   // 0, 1, 2, 3, 4
        p[idx] = (uint8_t)(code[v < 0 ? -v : v] | (v < 0 ? 0x80 : 0));
        return;
    }
    uint16_t h;
    if (arith == AR_BF16) {
        static const uint16_t code[5] = {0x0000, 0x3F80, 0x4000, 0x4040, 0x4080};
        h = (uint16_t)(code[v < 0 ? -v : v] | (v < 0 ? 0x8000 : 0));
    } else {
        static const uint16_t code[5] = {0x0000, 0x3C00, 0x4000, 0x4200, 0x4400};
        h = (uint16_t)(code[v < 0 ? -v : v] | (v < 0 ? 0x8000 : 0));
    }
    std::memcpy(p + 2 * idx, &h, 2);
}

}  // namespace

QGEMM_EXPORT int qgemm_selftest_layouts(char *buf, size_t buflen) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    int st = ensure_init_locked();
    if (st != QGEMM_OK) return st;
    std::string rep;
    bool all_ok = true;
    char line[256];

    // ---- LDS DMA: lane l's 16 bytes land at lds_base + 16*l, for low and high LDS addresses;
    //      out-of-range lanes write zeros
    {
        const int nsrc = 4096;
        std::vector<uint8_t> hsrc(nsrc);
        for (int i = 0; i < nsrc; ++i) hsrc[i] = (uint8_t)((i * 7 + (i >> 8)) & 0xFF);
        std::vector<uint32_t> hoff(64);
        for (int l = 0; l < 64; ++l) hoff[l] = (uint32_t)(((63 - l) * 48) % 2048);   // a permutation-ish gather, 16-aligned
        hoff[5] = 4096 + 64;   // out of range
        hoff[40] = 0xFFFFFF00u;
        hoff[7] = 3488;        // in range alone, out of range once soffset = 1024 is added
        void *dsrc = nullptr, *doff = nullptr, *dout = nullptr;
        HIP_TRY(hipMalloc(&dsrc, nsrc + 4096));   // slack behind the 4096-byte buffer range the probe declares
        HIP_TRY(hipMalloc(&doff, 256));
        HIP_TRY(hipMalloc(&dout, 1024));
        HIP_TRY(hipMemcpy(dsrc, hsrc.data(), nsrc, hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(doff, hoff.data(), 256, hipMemcpyHostToDevice));
        HIP_TRY(hipFuncSetAttribute((const void *)probe_lds_dma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    160 * 1024));
        const uint32_t bases[3] = {0, 72 * 1024, 159 * 1024};
        const uint32_t soffs[3] = {0, 1024, 16};
        for (int t = 0; t < 3; ++t) {
            hipLaunchKernelGGL(probe_lds_dma_kernel, dim3(1), dim3(64), 160 * 1024, 0, (const char *)dsrc,
                               (const uint32_t *)doff, (uint32_t)nsrc, bases[t], soffs[t], (char *)dout);
            HIP_TRY(hipGetLastError());
            std::vector<uint8_t> hout(1024);
            HIP_TRY(hipMemcpy(hout.data(), dout, 1024, hipMemcpyDeviceToHost));
            int bad = 0, oob_zero = 0, oob_untouched = 0;
            for (int l = 0; l < 64; ++l) {
                const uint64_t off = (uint64_t)hoff[l] + soffs[t];
                if (l == 7 && off + 16 > (uint64_t)nsrc) {
                    bool z = true;
                    for (int j = 0; j < 16; ++j) z &= hout[l * 16 + j] == 0;
                    std::snprintf(line, sizeof(line), "lds_dma: soffset %s part of the buffer range check\n",
                                  z ? "IS" : "is NOT");
                    rep += line;
                    // tile rows past M or N are kept out of reach by the range check alone (the row block of a
                    // copy sits in the scalar offset in the simple pipeline)
                    if (!z) all_ok = false;
                    continue;
                }
                if (off + 16 > (uint64_t)nsrc) {
                    bool z = true, u = true;
                    for (int j = 0; j < 16; ++j) {
                        z &= hout[l * 16 + j] == 0;
                        u &= hout[l * 16 + j] == 0xA5;
                    }
                    oob_zero += z;
                    oob_untouched += u;
                    continue;
                }
                for (int j = 0; j < 16; ++j) bad += hout[l * 16 + j] != hsrc[off + j];
            }
            std::snprintf(line, sizeof(line), "lds_dma base=%u soffset=%u: mismatched_bytes=%d oob_lanes_zero=%d oob_lanes_untouched=%d\n",
                          bases[t], soffs[t], bad, oob_zero, oob_untouched);
            rep += line;
            if (bad) all_ok = false;
        }
        (void)hipFree(dsrc);
        (void)hipFree(doff);
        (void)hipFree(dout);
    }

    // ---- 8-byte buffer loads at 4-byte aligned offsets, and across the end of the buffer range: the twin kernels
    //      for K-contiguous a_scale (two K blocks per load) read rows with an odd number of K blocks that way
    {
        const int n_in = 60;                                 // floats inside the range; 64 are allocated
        std::vector<float> h(64);
        for (int i = 0; i < 64; ++i) h[i] = 100.0f + (float)i;
        void *d = nullptr, *o = nullptr;
        HIP_TRY(hipMalloc(&d, 64 * 4));
        HIP_TRY(hipMalloc(&o, 128 * 4));
        HIP_TRY(hipMemcpy(d, h.data(), 64 * 4, hipMemcpyHostToDevice));
        hipLaunchKernelGGL(probe_b64_load_kernel, dim3(1), dim3(64), 0, 0, (const float *)d, (uint32_t)(n_in * 4), (int *)o);
        HIP_TRY(hipGetLastError());
        std::vector<float> got(128);
        HIP_TRY(hipMemcpy(got.data(), o, 128 * 4, hipMemcpyDeviceToHost));
        int bad = 0;
        for (int l = 0; l + 1 < n_in; ++l) bad += got[2 * l] != h[l] || got[2 * l + 1] != h[l + 1];
        const bool per_dword = got[2 * (n_in - 1)] == h[n_in - 1] && got[2 * (n_in - 1) + 1] == 0.0f;
        bool beyond_zero = true;
        for (int l = n_in; l < 64; ++l) beyond_zero &= got[2 * l] == 0.0f && got[2 * l + 1] == 0.0f;
        std::snprintf(line, sizeof(line), "b64 buffer load: mismatched_pairs=%d (odd lanes are 4-byte aligned only), range check %s, past_range_zero=%d\n",
                      bad, per_dword ? "per dword" : "NOT per dword", (int)beyond_zero);
        rep += line;
        if (bad || !per_dword || !beyond_zero) all_ok = false;
        (void)hipFree(d);
        (void)hipFree(o);
    }

    // ---- MFMA operand / accumulator layout for the four families
    {
        void *dx = nullptr, *dy = nullptr, *dout = nullptr;
        HIP_TRY(hipMalloc(&dx, 2048));
        HIP_TRY(hipMalloc(&dy, 2048));
        HIP_TRY(hipMalloc(&dout, 1024));
        const char *names[4] = {"i8", "f8", "bf16", "f16"};
        for (int arith = 0; arith < 4; ++arith) {
            const int eb = arith <= AR_F8 ? 1 : 2;
            const int per_lane = 32 / eb;                    // elements per lane per operand
            std::vector<uint8_t> hx(2048), hy(2048);
            uint32_t rng = 12345u + arith;
            auto next = [&]() { rng = rng * 1664525u + 1013904223u; return (int)((rng >> 24) % 9) - 4; };
            for (int i = 0; i < 64 * per_lane; ++i) {
                host_encode_small(arith, next(), hx.data(), i);
                host_encode_small(arith, next(), hy.data(), i);
            }
            HIP_TRY(hipMemcpy(dx, hx.data(), 2048, hipMemcpyHostToDevice));
            HIP_TRY(hipMemcpy(dy, hy.data(), 2048, hipMemcpyHostToDevice));
            switch (arith) {
                case AR_I8: hipLaunchKernelGGL(probe_mfma_kernel<AR_I8>, dim3(1), dim3(64), 0, 0, (const char *)dx, (const char *)dy, (int *)dout); break;
                case AR_F8: hipLaunchKernelGGL(probe_mfma_kernel<AR_F8>, dim3(1), dim3(64), 0, 0, (const char *)dx, (const char *)dy, (int *)dout); break;
                case AR_BF16: hipLaunchKernelGGL(probe_mfma_kernel<AR_BF16>, dim3(1), dim3(64), 0, 0, (const char *)dx, (const char *)dy, (int *)dout); break;
                default: hipLaunchKernelGGL(probe_mfma_kernel<AR_F16>, dim3(1), dim3(64), 0, 0, (const char *)dx, (const char *)dy, (int *)dout); break;
            }
            HIP_TRY(hipGetLastError());
            std::vector<int> hout(256);
            HIP_TRY(hipMemcpy(hout.data(), dout, 1024, hipMemcpyDeviceToHost));
            // assumed: operand lane l = row (l & 15), K group (l >> 4); the same element position of
            // the two operands meets in the contraction; accumulator lane l, register r =
            // D[first-operand row 4*(l >> 4) + r][second-operand row (l & 15)]
            int bad = 0;
            for (int l = 0; l < 64; ++l)
                for (int r = 0; r < 4; ++r) {
                    const int i = 4 * (l >> 4) + r, j = l & 15;
                    double sum = 0;
                    for (int g = 0; g < 4; ++g)
                        for (int e = 0; e < per_lane; ++e)
                            sum += (double)host_decode(arith, hx.data(), (g * 16 + i) * per_lane + e) *
                                   (double)host_decode(arith, hy.data(), (g * 16 + j) * per_lane + e);
                    double got;
                    if (arith == AR_I8) got = (double)hout[l * 4 + r];
                    else {
                        float f;
                        std::memcpy(&f, &hout[l * 4 + r], 4);
                        got = (double)f;
                    }
                    bad += got != sum;
                }
            std::snprintf(line, sizeof(line), "mfma %s: mismatched_accumulators=%d of 256\n", names[arith], bad);
            rep += line;
            if (bad) all_ok = false;
        }
        (void)hipFree(dx);
        (void)hipFree(dy);
        (void)hipFree(dout);
    }
    // ---- which XCD does workgroup i land on?  The tile raster assumes i % 8.
    {
        const int nwg = 64;
        void *dout = nullptr;
        HIP_TRY(hipMalloc(&dout, nwg * 8));
        hipLaunchKernelGGL(probe_xcc_kernel, dim3(nwg), dim3(64), 0, 0, (uint32_t *)dout);
        HIP_TRY(hipGetLastError());
        std::vector<uint32_t> h(nwg * 2);
        HIP_TRY(hipMemcpy(h.data(), dout, nwg * 8, hipMemcpyDeviceToHost));
        (void)hipFree(dout);
        int round_robin = 0;
        rep += "xcc of workgroups 0..31:";
        for (int i = 0; i < nwg; ++i) {
            if (i < 32) {
                std::snprintf(line, sizeof(line), " %u", h[i * 2] & 15u);
                rep += line;
            }
            round_robin += (int)(h[i * 2] & 15u) == i % kXcds;
        }
        std::snprintf(line, sizeof(line), "\nxcc round robin (wg %% 8): %d of %d workgroups\n", round_robin, nwg);
        rep += line;
    }
    if (buf && buflen) std::snprintf(buf, buflen, "%s", rep.c_str());
    return all_ok ? QGEMM_OK : QGEMM_ERR_UNSUPPORTED;
}

}  // extern "C"
