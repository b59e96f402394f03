// api.hip — the C ABI of include/larql_hip.h: context, weight residency, the
// host tier (trait-shaped calls on host slices) and the device tier.
//
// There is no CPU compute path in this library: every entry point either runs
// the HIP kernels or refuses.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/larql_hip.h"
#include "kernels.h"

using namespace larql;

// Scratch memory of larql_hip_dev_gate_knn_static, the entry point that allocates nothing: the score matrix, the hit
// counts and (Q4_0 gates) the quantised activation live here instead of in caller-provided or per-context buffers.
// Every GPU holds its own copy of the array; host code reaches it only through the address hipGetSymbolAddress
// returns for the current device (larql_hip_create keeps it in the context), never through the array's name.
// Layout: [scores: MAX_SCORES f32][counts: MAX_BATCH u32, padded to 256 B][Q8 codes: MAX_BATCH*MAX_HIDDEN i8]
//         [Q8 block scales: MAX_BATCH*MAX_HIDDEN/32 f32]
constexpr size_t kStaticScoresBytes = (size_t)LARQL_HIP_STATIC_MAX_SCORES * 4;
constexpr size_t kStaticCountsBytes = 256;
constexpr size_t kStaticQ8Bytes = (size_t)LARQL_HIP_STATIC_MAX_BATCH * LARQL_HIP_STATIC_MAX_HIDDEN;
constexpr size_t kStaticQ8ScaleBytes = kStaticQ8Bytes / 32 * 4;
constexpr size_t kStaticScratchBytes = kStaticScoresBytes + kStaticCountsBytes + kStaticQ8Bytes + kStaticQ8ScaleBytes;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Clears a few words on the stream (a kernel, not hipMemsetAsync: memset nodes recorded into a captured graph have
// given wrong results on replays).
// out[i] = parts[0][i] + parts[1][i] + ... (left to right), the partial vectors `stride` floats apart; up to eight
// such sums per launch (blockIdx.y says which)
constexpr int kSumBatch = 8;
struct SumPartialsArgs {
    const float *parts[kSumBatch];
    float *out[kSumBatch];
    uint32_t stride[kSumBatch], n_parts[kSumBatch], n[kSumBatch];
};
__global__ void sum_partials_kernel(SumPartialsArgs a) {
    const uint32_t q = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n[q]) return;
    const float *parts = a.parts[q];
    float acc = parts[i];
    for (uint32_t p = 1; p < a.n_parts[q]; p++) acc += parts[(size_t)p * a.stride[q] + i];
    a.out[q][i] = acc;
}

__global__ void zero_words_kernel(uint32_t *p, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

namespace {

struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
};

struct Region {
    const uint8_t *host;
    size_t len;
    uint8_t *dev;
};

// Page-locked host memory the device can address: small activations go up through it (an asynchronous copy from
// page-locked memory does not wait for a staging copy inside the runtime) and small results are WRITTEN into it by
// the kernels themselves, which spares a host-tier call the copy back.
struct PinBuf {
    void *host = nullptr, *dev = nullptr;
    size_t cap = 0;
};

}  // namespace

constexpr size_t kHostMats = 8;  // matrices one host-tier submission stages (their jobs travel in the kernel arguments)

// Job tables of host-tier and enqueue-only calls live in a few device buffers with pinned staging beside them; a call's
// table goes to the slot its shape hashes to, so that the calls of a loop (a layer's router gemv, gate/up and down
// launches, every token) each find the table they sent last time still in place.
constexpr int kTableSlots = 8;

struct larql_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    int cu_count = 0;
    int wgs_per_cu = 2;
    size_t flop_threshold = 500000000;  // the Metal peer's default (calibration.rs:12)
    std::mutex mu;
    std::string name, info, last_error;
    std::vector<Region> regions;
    DevBuf w[kHostMats], aux[kHostMats], x, out, tables[kTableSlots], misc, scores, q8, q8s, parts;
    // pinned staging for job tables: the upload is asynchronous, the event says when a slot may be rewritten
    void *table_host[kTableSlots] = {};
    size_t table_host_cap[kTableSlots] = {};
    hipEvent_t table_ev[kTableSlots] = {};
    void *table_sent_dst[kTableSlots] = {};   // where the table staged in table_host[i] went, and its size:
    size_t table_sent_bytes[kTableSlots] = {};  // an identical table for the same place is not sent again
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    uint8_t *log2_up = nullptr;  // 256-entry table for the MXFP4 encoder
    int *nan_flag = nullptr;       // [0]: device tier, raised by any call, cleared when taken; [1]: host tier, cleared by every call
    uint8_t *static_scratch = nullptr;  // this device's copy of `scratch` (hipGetSymbolAddress at create)
    larql_hip_submission_clock clock = {0, 0, 0};
    PinBuf pin_up, pin_out;   // host tier: activations on their way up (a ring, see upload()), results written by kernels
    size_t pin_up_off = 0, pin_up_call = 0;  // next free byte of the ring; bytes staged since the stream was last waited for
    // Times a call took device memory, staged a host buffer or uploaded a job table (larql_hip_debug_alloc_events):
    // what the entry point that allocates nothing must never do.
    uint64_t alloc_events = 0;
};

namespace {

int fail(larql_hip_ctx *c, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (c) c->last_error = buf;
    return code;
}

#define HIPCHECK(ctx, expr)                                                                         \
    do {                                                                                            \
        hipError_t _e = (expr);                                                                     \
        if (_e != hipSuccess) return fail(ctx, LARQL_E_DEVICE, "%s: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

int ensure(larql_hip_ctx *c, DevBuf &b, size_t bytes) {
    c->alloc_events++;  // (counted whether or not the buffer has to grow: the caller went through the staging path)
    if (bytes <= b.cap) return LARQL_OK;
    if (b.p) HIPCHECK(c, hipFree(b.p));
    b.p = nullptr; b.cap = 0;
    size_t cap = bytes < 4096 ? 4096 : bytes;
    HIPCHECK(c, hipMalloc(&b.p, cap));
    b.cap = cap;
    return LARQL_OK;
}

// A weight slice is served from a registered region when it lies inside one at
// a 16-byte aligned offset; otherwise it is uploaded into `staging` for the call.
int resolve_weights(larql_hip_ctx *c, const uint8_t *host, size_t len, DevBuf &staging, const uint8_t **dev) {
    for (const Region &r : c->regions) {
        if (host >= r.host && host + len <= r.host + r.len && ((size_t)(host - r.host) % 16) == 0) {
            *dev = r.dev + (host - r.host);
            return LARQL_OK;
        }
    }
    // pad so kernels that read an aligned window past the last block stay in bounds
    int rc = ensure(c, staging, len + 64);
    if (rc) return rc;
    if (len) HIPCHECK(c, hipMemcpyAsync(staging.p, host, len, hipMemcpyHostToDevice, c->stream));
    *dev = (const uint8_t *)staging.p;
    return LARQL_OK;
}

constexpr size_t kPinUpBytes = 4u << 20;    // the ring activations go up through
constexpr size_t kPinSmall = 512u << 10;    // what counts as small enough for page-locked staging / results

int ensure_pinned(larql_hip_ctx *c, PinBuf &b, size_t bytes) {
    if (bytes <= b.cap) return LARQL_OK;
    c->alloc_events++;
    if (b.host) {
        HIPCHECK(c, hipStreamSynchronize(c->stream));
        HIPCHECK(c, hipHostFree(b.host));
    }
    b.host = b.dev = nullptr; b.cap = 0;
    const size_t cap = bytes < 65536 ? 65536 : bytes;
    HIPCHECK(c, hipHostMalloc(&b.host, cap, hipHostMallocDefault));
    if (hipHostGetDevicePointer(&b.dev, b.host, 0) != hipSuccess || !b.dev) {
        (void)hipHostFree(b.host);
        b.host = nullptr;
        return fail(c, LARQL_E_DEVICE, "page-locked memory is not addressable by the device");
    }
    b.cap = cap;
    return LARQL_OK;
}

// Every host-tier call ends by waiting for the stream; from then on the whole ring is free again.
void stream_waited(larql_hip_ctx *c) { c->pin_up_call = 0; }
hipError_t wait_stream(larql_hip_ctx *c) {
    const hipError_t e = hipStreamSynchronize(c->stream);
    stream_waited(c);
    return e;
}

int upload(larql_hip_ctx *c, DevBuf &b, const void *host, size_t bytes) {
    int rc = ensure(c, b, bytes + 64);
    if (rc) return rc;
    if (!bytes) return LARQL_OK;
    // small: through the page-locked ring (slices of one call never overlap: a call that stages more than the ring
    // holds before it waits for the stream takes the pageable path for the rest)
    const size_t slice = (bytes + 255) & ~(size_t)255;
    if (bytes <= kPinSmall && c->pin_up_call + slice <= kPinUpBytes && ensure_pinned(c, c->pin_up, kPinUpBytes) == LARQL_OK) {
        if (c->pin_up_off + slice > kPinUpBytes) c->pin_up_off = 0;
        uint8_t *stage = (uint8_t *)c->pin_up.host + c->pin_up_off;
        memcpy(stage, host, bytes);
        c->pin_up_off += slice;
        c->pin_up_call += slice;
        HIPCHECK(c, hipMemcpyAsync(b.p, stage, bytes, hipMemcpyHostToDevice, c->stream));
        return LARQL_OK;
    }
    HIPCHECK(c, hipMemcpyAsync(b.p, host, bytes, hipMemcpyHostToDevice, c->stream));
    return LARQL_OK;
}

struct Submission {
    larql_hip_ctx *c;
    std::chrono::steady_clock::time_point t0;
    explicit Submission(larql_hip_ctx *ctx) : c(ctx), t0(std::chrono::steady_clock::now()) {
        (void)hipEventRecord(c->ev0, c->stream);
    }
    int finish() {
        HIPCHECK(c, hipEventRecord(c->ev1, c->stream));
        HIPCHECK(c, wait_stream(c));
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, c->ev0, c->ev1) == hipSuccess) c->clock.gpu_nanos += (uint64_t)(ms * 1e6);
        c->clock.submissions += 1;
        c->clock.commit_to_done_nanos += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
                                             std::chrono::steady_clock::now() - t0).count();
        return LARQL_OK;
    }
};

int kind_of_format(int format) {
    switch (format) {
        case LARQL_FMT_Q4_K: case LARQL_FMT_Q4_KF: return KIND_Q4K;
        case LARQL_FMT_GGML_Q8_0: return KIND_Q8_0;
        case LARQL_FMT_Q6_K: return KIND_Q6K;
        case LARQL_FMT_Q4_K_Q8K: return KIND_Q4K_Q8K;
        case LARQL_FMT_Q6_K_Q8K: return KIND_Q6K_Q8K;
        case LARQL_FMT_MXFP4: return KIND_MXFP4;
        case LARQL_FMT_Q4_0: return KIND_Q4_0;
        case LARQL_FMT_BF16: return KIND_BF16;
        case LARQL_FMT_F16: return KIND_F16;
        case LARQL_FMT_F32: return KIND_F32;
        default: return -1;
    }
}

struct PreparedLaunch {
    int kind;
    GemvLaunch L;
    uint32_t threads, grid;
    size_t lds;
    void *table = nullptr;  // owned device table when the jobs do not fit inline (plans only)
};

// Geometry for one launch over jobs of a single format.  When the jobs do not fit
// inline the table is uploaded into `table_dst` (synchronously: the host vector may die).
// A device table's size: the jobs and the first job of up to kTableFirstMax workgroups' shares.
constexpr size_t kTableFirstMax = 4096;
static size_t table_bytes_for(size_t n_jobs) { return n_jobs * sizeof(GemvJob) + kTableFirstMax * sizeof(uint32_t); }

int prepare_same_kind(larql_hip_ctx *c, GemvJob *live, size_t n_live, void *table_dst, PreparedLaunch &P, int stage_slot = -1) {
    P.kind = live[0].kind;
    P.threads = gemv_pick_threads(live, n_live);
    if (P.threads == 0) return fail(c, LARQL_UNSUPPORTED, "matvec: row length not supported by the gfx950 kernels");
    uint64_t total = 0;
    for (size_t ji = 0; ji < n_live; ji++) {
        GemvJob &j = live[ji];
        if (!gemv_job_geometry(j, P.threads)) return fail(c, LARQL_UNSUPPORTED, "matvec: unsupported geometry");
        if (total + j.n_pass > 0x7FFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "matvec: launch too large");
        j.pass_begin = (uint32_t)total;
        total += j.n_pass;
    }
    P.lds = gemv_lds_bytes(live, n_live, P.threads);
    uint64_t grid = (uint64_t)c->cu_count * (uint64_t)gemv_wgs_per_cu(P.kind, P.threads, P.lds, (uint32_t)c->wgs_per_cu);
    if (P.kind == KIND_Q4K_MFMA || P.kind == KIND_Q4K_Q8K) {
        // A launch with fewer 16-row tiles than workgroups: one workgroup per tile (and one more per job for its set-up
        // allowance), so that the tiles sit on consecutive workgroups — spread over the XCDs and CUs — and not on every
        // n-th one, where two of them can meet on a CU while others stand idle (a 3072 x 1024 matvec alone: 5.3 -> 4.3 us).
        uint64_t tiles = 0;
        for (size_t ji = 0; ji < n_live; ji++) tiles += (live[ji].rows + 15) / 16 + 1;
        if (grid > tiles) grid = tiles;
    }
    // the share-out's cost model wants to know how long a workgroup's share is: a second pass over the costs
    if (gemv_refine_costs(live, n_live, (uint32_t)std::min<uint64_t>(grid, 0xFFFFFFFFull))) {
        total = 0;
        for (size_t ji = 0; ji < n_live; ji++) {
            if (total + live[ji].n_pass > 0x7FFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "matvec: launch too large");
            live[ji].pass_begin = (uint32_t)total;
            total += live[ji].n_pass;
        }
    }
    if (grid > total) grid = total;
    P.grid = (uint32_t)grid;
    memset(&P.L, 0, sizeof P.L);
    P.L.total_passes = total;
    P.L.n_jobs = (uint32_t)n_live;
    P.L.pad = gemv_launch_param(live, n_live);
    if (n_live <= (size_t)kInlineJobs) {
        for (size_t i = 0; i < n_live; i++) P.L.inl[i] = live[i];
        P.L.table = nullptr;
    } else {
        // the table: the jobs, then the first job of every workgroup's share (what a workgroup would otherwise find by
        // bisection over the jobs' pass ranges, a dependent load per step)
        c->alloc_events++;
        const size_t job_bytes = n_live * sizeof(GemvJob);
        const bool with_first = grid >= 1 && grid <= (uint64_t)kTableFirstMax;
        const size_t bytes = job_bytes + (with_first ? (size_t)grid * sizeof(uint32_t) : 0);
        std::vector<uint8_t> blob(bytes);
        memcpy(blob.data(), live, job_bytes);
        if (with_first) {
            uint32_t *first = (uint32_t *)(blob.data() + job_bytes);
            size_t ji = 0;
            for (uint64_t b = 0; b < grid; b++) {
                const uint64_t pb = total * b / grid;
                while (ji + 1 < n_live && (uint64_t)live[ji + 1].pass_begin <= pb) ji++;
                first[b] = (uint32_t)ji;
            }
        }
        if (stage_slot >= 0 && c->table_sent_dst[stage_slot] == table_dst && c->table_sent_bytes[stage_slot] == bytes &&
            memcmp(c->table_host[stage_slot], blob.data(), bytes) == 0) {
            // the same jobs as the last call through this slot (a decode loop): the device table is already (or, in
            // stream order, about to be) what this launch needs
        } else if (stage_slot >= 0) {
            // through pinned memory: no host wait, the launch that follows on the stream sees the table
            c->table_sent_dst[stage_slot] = nullptr;
            if (c->table_host_cap[stage_slot] < bytes) {
                if (c->table_ev[stage_slot]) HIPCHECK(c, hipEventSynchronize(c->table_ev[stage_slot]));
                if (c->table_host[stage_slot]) HIPCHECK(c, hipHostFree(c->table_host[stage_slot]));
                c->table_host[stage_slot] = nullptr; c->table_host_cap[stage_slot] = 0;
                HIPCHECK(c, hipHostMalloc(&c->table_host[stage_slot], bytes * 2, hipHostMallocDefault));
                c->table_host_cap[stage_slot] = bytes * 2;
            }
            if (!c->table_ev[stage_slot]) HIPCHECK(c, hipEventCreateWithFlags(&c->table_ev[stage_slot], hipEventDisableTiming));
            else HIPCHECK(c, hipEventSynchronize(c->table_ev[stage_slot]));  // the previous upload from this slot is done
            memcpy(c->table_host[stage_slot], blob.data(), bytes);
            HIPCHECK(c, hipMemcpyAsync(table_dst, c->table_host[stage_slot], bytes, hipMemcpyHostToDevice, c->stream));
            HIPCHECK(c, hipEventRecord(c->table_ev[stage_slot], c->stream));
            c->table_sent_dst[stage_slot] = table_dst;
            c->table_sent_bytes[stage_slot] = bytes;
        } else {
            HIPCHECK(c, hipMemcpyAsync(table_dst, blob.data(), bytes, hipMemcpyHostToDevice, c->stream));
            HIPCHECK(c, wait_stream(c));  // the host vector may die
        }
        P.L.table = (const GemvJob *)table_dst;
        if (with_first) P.L.wg_first = (const uint32_t *)((const uint8_t *)table_dst + job_bytes);
    }
    return LARQL_OK;
}

int check_jobs(larql_hip_ctx *c, const std::vector<GemvJob> &jobs) {
    for (const GemvJob &j : jobs) {
        if (j.rows == 0) continue;
        if (((uintptr_t)j.w & 15) || ((uintptr_t)j.x & 15))
            return fail(c, LARQL_REFUSED_SHAPE, "matvec: weight and activation pointers must be 16-byte aligned");
    }
    return LARQL_OK;
}

// Split jobs into one group per format present, in first-seen order.
std::vector<std::vector<GemvJob>> group_by_kind(const std::vector<GemvJob> &jobs_in) {
    std::vector<GemvJob> jobs(jobs_in);
    for (GemvJob &j : jobs) j.kind = gemv_effective_kind(j);  // Q4_K rows the matrix-core kernel takes get their own launch
    std::vector<std::vector<GemvJob>> groups;
    bool done[16] = {};
    for (size_t i = 0; i < jobs.size(); i++) {
        const int kind = jobs[i].kind;
        if (jobs[i].rows == 0 || kind < 0 || kind > 15 || done[kind]) continue;
        done[kind] = true;
        std::vector<GemvJob> live;
        for (size_t t = i; t < jobs.size(); t++)
            if (jobs[t].kind == kind && jobs[t].rows > 0) live.push_back(jobs[t]);
        groups.push_back(live);
    }
    return groups;
}

// Q4_K rows longer than the matrix-core kernels take (40 super-blocks of 256) are served as column ranges of at most 40
// super-blocks: every range a job of its own over the rows of the full matrix (GemvJob::row_stride) into a partial
// vector of its own, the partial vectors added in range order by sum_partials_kernel.  The ranges of a row of `cpr`
// super-blocks, as {first super-block, count}: as few as fit, of equal length up to one super-block.
constexpr uint64_t kQ4kRangeMax = 40;
std::vector<std::pair<uint64_t, uint64_t>> q4k_row_ranges(uint64_t cpr) {
    std::vector<std::pair<uint64_t, uint64_t>> r;
    const uint64_t n = (cpr + kQ4kRangeMax - 1) / kQ4kRangeMax;
    uint64_t at = 0;
    for (uint64_t i = 0; i < n; i++) {
        const uint64_t len = cpr / n + (i < cpr % n ? 1 : 0);
        r.push_back({at, len});
        at += len;
    }
    return r;
}
// The device layout of a Q8_K activation whose row is served in ranges: range after range, each [codes | scales | sums]
// of its own and 64-byte aligned (the kernel finds a job's scales and sums behind its k codes).
size_t q8k_ranged_bytes(size_t cols) {
    size_t total = 0;
    for (const auto &rg : q4k_row_ranges(cols / 256)) total += (q8k_bytes(rg.second * 256) + 63) & ~(size_t)63;
    return total;
}
struct SplitSum { float *out; size_t parts_off, rows; uint32_t n_parts; };
// Replaces every plain Q4_K / Q4_K x Q8_K job with rows beyond the kernels' reach by its range jobs (a Q8_K activation
// must be laid out by q8k_ranged_bytes' rule); `sums` says what to add up afterwards, `parts_floats` how much room the
// partial vectors take.
bool split_long_q4k_rows(std::vector<GemvJob> &jobs, std::vector<SplitSum> &sums, size_t &parts_floats) {
    std::vector<GemvJob> outj;
    parts_floats = 0;
    bool any = false;
    for (const GemvJob &j : jobs) {
        // (f32 activations: rows of up to 128 super-blocks have the K-slice kernel — one launch, no partial sums, and
        // measured no slower than ranges plus their addition; the Q8_K kernel has no other way beyond 40)
        const uint64_t reach = j.kind == KIND_Q4K ? 128 : kQ4kRangeMax;
        const bool long_row = (j.kind == KIND_Q4K || j.kind == KIND_Q4K_Q8K) && j.k % 256 == 0 && j.k / 256 > reach && j.rows > 0 &&
                              !j.sel && j.batch <= 1 && !j.bias && !j.row_stride && (j.k / 256) * 144 <= (1ull << 27);
        if (!long_row) { outj.push_back(j); continue; }
        any = true;
        const auto ranges = q4k_row_ranges(j.k / 256);
        const size_t rows_up = ((size_t)j.rows + 63) & ~(size_t)63;
        sums.push_back({j.out, parts_floats, (size_t)j.rows, (uint32_t)ranges.size()});
        size_t q8_off = 0;
        for (size_t i = 0; i < ranges.size(); i++) {
            GemvJob s = j;
            s.w = j.w + ranges[i].first * 144;
            s.row_stride = (j.k / 256) * 144;
            s.k = ranges[i].second * 256;
            if (j.kind == KIND_Q4K) s.x = j.x + ranges[i].first * 256;
            else { s.x = (const float *)((const uint8_t *)j.x + q8_off); q8_off += (q8k_bytes(s.k) + 63) & ~(size_t)63; }
            s.out = reinterpret_cast<float *>((uintptr_t)((parts_floats + i * rows_up) * sizeof(float)));  // (a byte offset into the partial area: rebased by the caller)
            outj.push_back(s);
        }
        parts_floats += ranges.size() * rows_up;
    }
    if (any) jobs.swap(outj);
    return any;
}

// Enqueue `jobs` (device operands): one launch per format present, in first-seen
// order.  Jobs with no rows are dropped.
int enqueue_jobs(larql_hip_ctx *c, std::vector<GemvJob> &jobs_in) {
    std::vector<GemvJob> jobs(jobs_in);
    std::vector<SplitSum> sums;
    size_t parts_floats = 0;
    if (split_long_q4k_rows(jobs, sums, parts_floats)) {
        int rc0 = ensure(c, c->parts, parts_floats * sizeof(float) + 64);
        if (rc0) return rc0;
        for (GemvJob &j : jobs)
            if (j.row_stride) j.out = reinterpret_cast<float *>((uint8_t *)c->parts.p + reinterpret_cast<uintptr_t>(j.out));
    }
    int rc = check_jobs(c, jobs);
    if (rc) return rc;
    for (std::vector<GemvJob> &live : group_by_kind(jobs)) {
        const int sl = (int)(((size_t)live[0].kind * 31 + live.size() * 7 + ((uintptr_t)live[0].w >> 8) + ((uintptr_t)live[0].out >> 6)) % kTableSlots);
        DevBuf &tb = c->tables[sl];
        if (live.size() > (size_t)kInlineJobs) {
            const void *before = tb.p;
            rc = ensure(c, tb, table_bytes_for(live.size()));
            if (rc) return rc;
            if (tb.p != before) c->table_sent_dst[sl] = nullptr;  // a new allocation holds nothing yet
        }
        PreparedLaunch P;
        rc = prepare_same_kind(c, live.data(), live.size(), tb.p, P, sl);
        if (rc) return rc;
        HIPCHECK(c, gemv_launch(c->stream, P.kind, P.L, P.threads, P.grid, P.lds));
    }
    for (size_t at = 0; at < sums.size(); at += kSumBatch) {
        SumPartialsArgs a;
        memset(&a, 0, sizeof a);
        const size_t nb = std::min<size_t>(kSumBatch, sums.size() - at);
        size_t longest = 0;
        for (size_t q = 0; q < nb; q++) {
            const SplitSum &sm = sums[at + q];
            if (sm.rows > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "matvec: too many rows");
            a.parts[q] = (const float *)c->parts.p + sm.parts_off;
            a.out[q] = sm.out;
            a.stride[q] = (uint32_t)((sm.rows + 63) & ~(size_t)63);
            a.n_parts[q] = sm.n_parts;
            a.n[q] = (uint32_t)sm.rows;
            longest = std::max(longest, sm.rows);
        }
        hipLaunchKernelGGL(sum_partials_kernel, dim3((unsigned)((longest + 255) / 256), (unsigned)nb), dim3(256), 0, c->stream, a);
        HIPCHECK(c, hipGetLastError());
    }
    return LARQL_OK;
}

GemvJob make_job(int kind, const void *w, const void *aux, const void *x, float *out, uint64_t rows, uint64_t k) {
    GemvJob j;
    memset(&j, 0, sizeof j);
    j.kind = kind; j.w = (const uint8_t *)w; j.aux = (const uint8_t *)aux; j.x = (const float *)x; j.out = out;
    j.rows = rows; j.k = k;
    return j;
}

size_t dense_elem_bytes(int kind) { return kind == KIND_F32 ? 4 : 2; }

}  // namespace

extern "C" {

// ---- lifecycle ----------------------------------------------------------------
int larql_hip_create(larql_hip_ctx **out, int device) {
    if (!out) return LARQL_E_ARG;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0 || device < 0 || device >= n) return LARQL_E_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return LARQL_E_NO_DEVICE;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return LARQL_E_NO_DEVICE;  // code objects are gfx950 only
    if (hipSetDevice(device) != hipSuccess) return LARQL_E_NO_DEVICE;
    larql_hip_ctx *c = new larql_hip_ctx();
    c->device = device;
    c->cu_count = prop.multiProcessorCount;
    char buf[256];
    snprintf(buf, sizeof buf, "hip (gfx950 matvec + gate-KNN kernels)");
    c->name = buf;
    snprintf(buf, sizeof buf, "%s, %d CUs, %.0f GiB HBM, %s", prop.name[0] ? prop.name : "AMD Instinct (gfx950)", prop.multiProcessorCount,
             (double)prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0), prop.gcnArchName);
    c->info = buf;
    if (hipStreamCreate(&c->stream) != hipSuccess || hipEventCreate(&c->ev0) != hipSuccess ||
        hipEventCreate(&c->ev1) != hipSuccess || hipMalloc((void **)&c->log2_up, 256) != hipSuccess ||
        hipMalloc((void **)&c->nan_flag, 2 * sizeof(int)) != hipSuccess) {
        larql_hip_destroy(c);
        return LARQL_E_DEVICE;
    }
    // For each f32 exponent E: how many of the largest mantissas have a host
    // log2f that rounds up to the next integer (the MXFP4 encoder's floor(log2f)).
    uint8_t up[256];
    for (int E = 0; E < 256; E++) {
        up[E] = 0;
        if (E == 0 || E == 255) continue;
        for (uint32_t kk = 1; kk <= 64; kk++) {
            uint32_t bits = ((uint32_t)E << 23) | (0x800000u - kk);
            float v; memcpy(&v, &bits, 4);
            if (floorf(log2f(v)) == (float)(E - 127 + 1)) up[E] = (uint8_t)kk; else break;
        }
    }
    if (hipMemcpy(c->log2_up, up, 256, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemset(c->nan_flag, 0, 2 * sizeof(int)) != hipSuccess) {
        larql_hip_destroy(c);
        return LARQL_E_DEVICE;
    }
    // the address of this device's copy of the static scratch array (the device is current: hipSetDevice above)
    void *sp = nullptr;
    if (hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)) != hipSuccess || !sp) {
        larql_hip_destroy(c);
        return LARQL_E_DEVICE;
    }
    c->static_scratch = (uint8_t *)sp;
    *out = c;
    return LARQL_OK;
}

void larql_hip_destroy(larql_hip_ctx *c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (Region &r : c->regions) (void)hipFree(r.dev);
    DevBuf *bufs[] = {&c->x, &c->out, &c->misc, &c->scores, &c->q8, &c->q8s, &c->parts};
    for (DevBuf &t : c->tables) if (t.p) (void)hipFree(t.p);
    for (DevBuf *b : bufs) if (b->p) (void)hipFree(b->p);
    for (size_t i = 0; i < kHostMats; i++) {
        if (c->w[i].p) (void)hipFree(c->w[i].p);
        if (c->aux[i].p) (void)hipFree(c->aux[i].p);
    }
    for (int i = 0; i < kTableSlots; i++) {
        if (c->table_host[i]) (void)hipHostFree(c->table_host[i]);
        if (c->table_ev[i]) (void)hipEventDestroy(c->table_ev[i]);
    }
    if (c->pin_up.host) (void)hipHostFree(c->pin_up.host);
    if (c->pin_out.host) (void)hipHostFree(c->pin_out.host);
    if (c->log2_up) (void)hipFree(c->log2_up);
    if (c->nan_flag) (void)hipFree(c->nan_flag);
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

const char *larql_hip_name(const larql_hip_ctx *c) { return c ? c->name.c_str() : ""; }
const char *larql_hip_device_info(const larql_hip_ctx *c) { return c ? c->info.c_str() : ""; }
const char *larql_hip_last_error(const larql_hip_ctx *c) { return c ? c->last_error.c_str() : "null context"; }

int larql_hip_supports_quant(const larql_hip_ctx *, int format) {
    switch (format) {
        case LARQL_FMT_Q4_0: case LARQL_FMT_Q4_K: case LARQL_FMT_Q4_KF: case LARQL_FMT_Q6_K: case LARQL_FMT_MXFP4:
        case LARQL_FMT_GGML_Q8_0: case LARQL_FMT_BF16: case LARQL_FMT_F16: case LARQL_FMT_F32:
            return 1;
        default:
            return 0;
    }
}

int larql_hip_supports(const larql_hip_ctx *, int cap) {
    return cap == LARQL_CAP_F32_GEMV || cap == LARQL_CAP_F16_GEMV || cap == LARQL_CAP_QUANT_MATVEC;
}

int larql_hip_register_weight_region(larql_hip_ctx *c, const uint8_t *region, size_t len) {
    if (!c || (!region && len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    for (const Region &r : c->regions)
        if (r.host == region && r.len >= len) return LARQL_OK;  // same base twice: no-op
    if (len == 0) return LARQL_OK;
    Region r{region, len, nullptr};
    HIPCHECK(c, hipMalloc((void **)&r.dev, len + 64));
    hipError_t e = hipMemcpy(r.dev, region, len, hipMemcpyHostToDevice);
    if (e != hipSuccess) { (void)hipFree(r.dev); return fail(c, LARQL_E_DEVICE, "register_weight_region: %s", hipGetErrorString(e)); }
    c->regions.push_back(r);
    return LARQL_OK;
}

int larql_hip_seal_weight_regions(larql_hip_ctx *c) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipDeviceSynchronize());  // uploads are complete; nothing else to declare on this platform
    return LARQL_OK;
}

int larql_hip_clear_weight_regions(larql_hip_ctx *c) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, wait_stream(c));
    for (Region &r : c->regions) (void)hipFree(r.dev);
    c->regions.clear();
    return LARQL_OK;
}

int larql_hip_get_submission_clock(larql_hip_ctx *c, larql_hip_submission_clock *out) {
    if (!c || !out) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    *out = c->clock;
    return LARQL_OK;
}

// ---- host tier: quantised matvec -------------------------------------------------

// Where a host-tier call's f32 result goes: page-locked host memory the kernel writes itself when it is small
// (no copy back), the context's device buffer otherwise.
struct ResultArea {
    float *dev;
    bool direct;
};
static int result_area(larql_hip_ctx *c, size_t bytes, ResultArea &r) {
    r.direct = bytes <= kPinSmall && ensure_pinned(c, c->pin_out, kPinSmall + 64) == LARQL_OK;
    if (!r.direct) { int rc = ensure(c, c->out, bytes + 64); if (rc) return rc; }
    r.dev = (float *)(r.direct ? c->pin_out.dev : c->out.p);
    return LARQL_OK;
}
// ends the submission (one wait for the stream) and leaves the result in `dst`
static int finish_with_result(larql_hip_ctx *c, Submission &sub, const ResultArea &r, void *dst, size_t bytes) {
    if (!r.direct) HIPCHECK(c, hipMemcpyAsync(dst, r.dev, bytes, hipMemcpyDeviceToHost, c->stream));
    const int rc = sub.finish();
    if (rc == LARQL_OK && r.direct) memcpy(dst, c->pin_out.host, bytes);
    return rc;
}

static int host_matvec_multi(larql_hip_ctx *c, int kind, size_t n_mats, const uint8_t *const *w, const size_t *w_len,
                             const uint8_t *const *aux, const size_t *aux_len, const size_t *rows, size_t k,
                             const float *x, size_t x_bytes, float *const *out) {
    if (n_mats > kHostMats) return fail(c, LARQL_UNSUPPORTED, "at most %zu matrices per host-tier submission", kHostMats);
    HIPCHECK(c, hipSetDevice(c->device));
    std::vector<GemvJob> jobs;
    int rc = upload(c, c->x, x, x_bytes);
    if (rc) return rc;
    size_t out_total = 0;
    for (size_t i = 0; i < n_mats; i++) out_total += rows[i];
    // small results are written by the kernel straight into page-locked host memory: no copy back
    const bool direct = out_total * sizeof(float) <= kPinSmall && ensure_pinned(c, c->pin_out, kPinSmall + 64) == LARQL_OK;
    if (!direct) { rc = ensure(c, c->out, out_total * sizeof(float) + 64); if (rc) return rc; }
    float *d_out = direct ? (float *)c->pin_out.dev : (float *)c->out.p;
    size_t off = 0;
    for (size_t i = 0; i < n_mats; i++) {
        const uint8_t *dw = nullptr, *da = nullptr;
        rc = resolve_weights(c, w[i], w_len[i], c->w[i], &dw);
        if (rc) return rc;
        if (aux) { rc = resolve_weights(c, aux[i], aux_len[i], c->aux[i], &da); if (rc) return rc; }
        jobs.push_back(make_job(kind, dw, da, c->x.p, d_out + off, rows[i], k));
        off += rows[i];
    }
    Submission sub(c);
    rc = enqueue_jobs(c, jobs);
    if (rc) { (void)hipStreamSynchronize(c->stream); stream_waited(c); return rc; }
    off = 0;
    if (!direct)
        for (size_t i = 0; i < n_mats; i++) {
            if (rows[i]) HIPCHECK(c, hipMemcpyAsync(out[i], (float *)c->out.p + off, rows[i] * sizeof(float), hipMemcpyDeviceToHost, c->stream));
            off += rows[i];
        }
    rc = sub.finish();
    if (rc || !direct) return rc;
    for (size_t i = 0; i < n_mats; i++) {
        if (rows[i]) memcpy(out[i], (const float *)c->pin_out.host + off, rows[i] * sizeof(float));
        off += rows[i];
    }
    return LARQL_OK;
}

static bool q4k_shape_ok(size_t out_len, size_t rows, size_t x_len, size_t cols, size_t w_len) {
    // KernelShapeError::check, larql-compute/src/cpu/ops/kernel_shape.rs:46-75
    const size_t needed = (cols / 256) * 144 * rows;
    return out_len == rows && x_len == cols && cols % 256 == 0 && w_len >= needed;
}

int larql_hip_q4k_matvec(larql_hip_ctx *c, const uint8_t *q4k, size_t q4k_len, const float *x, size_t x_len,
                         size_t num_rows, size_t hidden, float *out, size_t out_len) {
    if (!c || (!out && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (!q4k_shape_ok(out_len, num_rows, x_len, hidden, q4k_len))
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_matvec: refused operands: out.len() %zu for %zu rows, activation length %zu for %zu cols, %zu weight bytes",
                    out_len, num_rows, x_len, hidden, q4k_len);
    if (num_rows == 0 || hidden == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q4k || !x) return LARQL_E_ARG;
    const size_t need = (hidden / 256) * 144 * num_rows;
    return host_matvec_multi(c, KIND_Q4K, 1, &q4k, &need, nullptr, nullptr, &num_rows, hidden, x, x_len * 4, &out);
}

int larql_hip_q6k_matvec(larql_hip_ctx *c, const uint8_t *q6k, size_t q6k_len, const float *x, size_t x_len, size_t num_rows,
                         size_t hidden, float *out) {
    if (!c || (!out && num_rows)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const size_t need = (hidden / 256) * 210 * num_rows;
    if (hidden % 256 != 0 || x_len != hidden || q6k_len < need)
        return fail(c, LARQL_REFUSED_SHAPE, "q6k_matvec: refused operands: activation length %zu for %zu cols, %zu weight bytes for %zu rows",
                    x_len, hidden, q6k_len, num_rows);
    if (num_rows == 0 || hidden == 0) { for (size_t i = 0; i < num_rows; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q6k || !x) return LARQL_E_ARG;
    return host_matvec_multi(c, KIND_Q6K, 1, &q6k, &need, nullptr, nullptr, &num_rows, hidden, x, x_len * 4, &out);
}

// ---- Q8_K-activation integer path (larql-compute/src/cpu/ops/q4k_q8k_dot) --------------------------------

size_t larql_hip_q8k_bytes(size_t n) { return q8k_bytes(n); }

int larql_hip_dev_quantize_x_to_q8k(larql_hip_ctx *c, const float *x, size_t n, void *q8k) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_x_to_q8k: length must be a multiple of 256");
    if (n == 0) return LARQL_OK;
    if (!x || !q8k || ((uintptr_t)x & 15) || ((uintptr_t)q8k & 15)) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_x_to_q8k_launch(c->stream, x, n, (uint8_t *)q8k));
    return LARQL_OK;
}

int larql_hip_quantize_x_to_q8k(larql_hip_ctx *c, const float *x, size_t n, int8_t *qs, float *d, int16_t *sums) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_x_to_q8k: length must be a multiple of 256");
    if (n == 0) return LARQL_OK;
    if (!x || !qs || !d || !sums) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    int rc = upload(c, c->x, x, n * 4);
    if (rc) return rc;
    rc = ensure(c, c->misc, q8k_bytes(n) + 64);
    if (rc) return rc;
    Submission sub(c);
    HIPCHECK(c, quantize_x_to_q8k_launch(c->stream, (const float *)c->x.p, n, (uint8_t *)c->misc.p));
    const uint8_t *p = (const uint8_t *)c->misc.p;
    HIPCHECK(c, hipMemcpyAsync(qs, p, n, hipMemcpyDeviceToHost, c->stream));
    HIPCHECK(c, hipMemcpyAsync(d, p + n, (n / 256) * 4, hipMemcpyDeviceToHost, c->stream));
    HIPCHECK(c, hipMemcpyAsync(sums, p + n + (n / 256) * 4, (n / 32) * 2, hipMemcpyDeviceToHost, c->stream));
    return sub.finish();
}

static void pack_q8k(uint8_t *dst, const int8_t *qs, const float *d, const int16_t *sums, size_t cols) {
    memcpy(dst, qs, cols);  // the activation travels in its device layout: [codes | scales | sums]
    memcpy(dst + cols, d, (cols / 256) * 4);
    memcpy(dst + cols + (cols / 256) * 4, sums, (cols / 32) * 2);
}
// ... range after range where the row is longer than one job takes (q8k_ranged_bytes; a row of up to 10240 elements is one range)
static std::vector<uint8_t> pack_q8k_ranged(const int8_t *qs, const float *d, const int16_t *sums, size_t cols) {
    std::vector<uint8_t> packed(q8k_ranged_bytes(cols), 0);
    size_t off = 0;
    for (const auto &rg : q4k_row_ranges(cols / 256)) {
        pack_q8k(packed.data() + off, qs + rg.first * 256, d + rg.first, sums + rg.first * 8, rg.second * 256);
        off += (q8k_bytes(rg.second * 256) + 63) & ~(size_t)63;
    }
    return packed;
}

int larql_hip_q4k_q8k_matvec(larql_hip_ctx *c, const uint8_t *q4k, size_t q4k_len, const int8_t *qs, size_t qs_len, const float *d,
                             const int16_t *sums, size_t num_rows, size_t cols, float *out, size_t out_len) {
    if (!c || (!out && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (!q4k_shape_ok(out_len, num_rows, qs_len, cols, q4k_len))
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_q8k_matvec: refused operands: out.len() %zu for %zu rows, activation length %zu for %zu cols, %zu weight bytes",
                    out_len, num_rows, qs_len, cols, q4k_len);
    if (num_rows == 0 || cols == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q4k || !qs || !d || !sums) return LARQL_E_ARG;
    if ((cols / 256) * 144 > (1ull << 27)) return fail(c, LARQL_UNSUPPORTED, "q4k_q8k_matvec: rows this long have no kernel");
    const std::vector<uint8_t> packed = pack_q8k_ranged(qs, d, sums, cols);
    const size_t need = (cols / 256) * 144 * num_rows;
    return host_matvec_multi(c, KIND_Q4K_Q8K, 1, &q4k, &need, nullptr, nullptr, &num_rows, cols, (const float *)packed.data(), packed.size(), &out);
}

int larql_hip_q4k_q8k_gate_up(larql_hip_ctx *c, const uint8_t *gate_w, size_t gate_len, const uint8_t *up_w, size_t up_len,
                              const int8_t *qs, size_t qs_len, const float *d, const int16_t *sums, size_t num_rows, size_t cols,
                              float *gate_out, float *up_out, size_t out_len) {
    if (!c || ((!gate_out || !up_out) && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    // both halves are checked before anything is written (gate_up.rs:68-87): a refusal touches neither output
    if (!q4k_shape_ok(out_len, num_rows, qs_len, cols, gate_len) || !q4k_shape_ok(out_len, num_rows, qs_len, cols, up_len))
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_q8k_gate_up: refused operands: out.len() %zu for %zu rows, activation length %zu for %zu cols, %zu / %zu weight bytes",
                    out_len, num_rows, qs_len, cols, gate_len, up_len);
    if (num_rows == 0 || cols == 0) { for (size_t i = 0; i < out_len; i++) { gate_out[i] = 0.0f; up_out[i] = 0.0f; } return LARQL_OK; }
    if (!gate_w || !up_w || !qs || !d || !sums) return LARQL_E_ARG;
    if ((cols / 256) * 144 > (1ull << 27)) return fail(c, LARQL_UNSUPPORTED, "q4k_q8k_gate_up: rows this long have no kernel");
    const std::vector<uint8_t> packed = pack_q8k_ranged(qs, d, sums, cols);
    const size_t need = (cols / 256) * 144 * num_rows;
    const uint8_t *w[2] = {gate_w, up_w};
    const size_t needs[2] = {need, need}, rows[2] = {num_rows, num_rows};
    float *outs[2] = {gate_out, up_out};
    return host_matvec_multi(c, KIND_Q4K_Q8K, 2, w, needs, nullptr, nullptr, rows, cols, (const float *)packed.data(), packed.size(), outs);
}

int larql_hip_q4k_q8k_gemm(larql_hip_ctx *c, const uint8_t *q4k, size_t q4k_len, const int8_t *qs, const float *d, const int16_t *sums,
                           size_t seq, size_t num_rows, size_t cols, float *out, size_t out_len) {
    if (!c || (!out && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const size_t need = (cols / 256) * 144 * num_rows;
    if (out_len != seq * num_rows || cols % 256 != 0 || q4k_len < need)  // (the reference asserts these)
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_q8k_gemm: refused operands: out.len() %zu for %zu x %zu, %zu cols, %zu weight bytes", out_len, seq,
                    num_rows, cols, q4k_len);
    if (seq == 0 || num_rows == 0) return LARQL_OK;
    if (cols == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q4k || !qs || !d || !sums) return LARQL_E_ARG;
    if (cols / 256 > 40) return fail(c, LARQL_UNSUPPORTED, "q4k_q8k_gemm: rows longer than 10240 have no kernel");
    if (seq > 65536) return fail(c, LARQL_UNSUPPORTED, "q4k_q8k_gemm: more than 65536 activation rows");
    HIPCHECK(c, hipSetDevice(c->device));
    // one launch: a job per activation row against the one resident copy of the weights (the reference runs the
    // row-at-a-time kernel per activation row and holds the result to it bit for bit)
    const size_t stride = (q8k_bytes(cols) + 63) & ~(size_t)63;
    std::vector<uint8_t> packed(stride * seq);
    for (size_t s = 0; s < seq; s++)
        pack_q8k(packed.data() + s * stride, qs + s * cols, d + s * (cols / 256), sums + s * (cols / 32), cols);
    int rc = upload(c, c->x, (const float *)packed.data(), packed.size());
    if (rc) return rc;
    ResultArea res;
    rc = result_area(c, out_len * sizeof(float), res);
    if (rc) return rc;
    const uint8_t *dw = nullptr;
    rc = resolve_weights(c, q4k, need, c->w[0], &dw);
    if (rc) return rc;
    std::vector<GemvJob> jobs;
    jobs.reserve(seq);
    for (size_t s = 0; s < seq; s++)
        jobs.push_back(make_job(KIND_Q4K_Q8K, dw, nullptr, (const uint8_t *)c->x.p + s * stride, res.dev + s * num_rows, num_rows, cols));
    Submission sub(c);
    rc = enqueue_jobs(c, jobs);
    if (rc) { (void)wait_stream(c); return rc; }
    return finish_with_result(c, sub, res, out, out_len * sizeof(float));
}

int larql_hip_q6k_q8k_matvec(larql_hip_ctx *c, const uint8_t *q6k, size_t q6k_len, const int8_t *qs, size_t qs_len, const float *d,
                             size_t num_rows, size_t cols, float *out, size_t out_len) {
    if (!c || (!out && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    // KernelShapeError::check with 210-byte blocks (cpu/ops/q4k_q8k_dot/q6k.rs:15-36)
    const size_t need = (cols / 256) * 210 * num_rows;
    if (out_len != num_rows || qs_len != cols || cols % 256 != 0 || q6k_len < need)
        return fail(c, LARQL_REFUSED_SHAPE, "q6k_q8k_matvec: refused operands: out.len() %zu for %zu rows, activation length %zu for %zu cols, %zu weight bytes",
                    out_len, num_rows, qs_len, cols, q6k_len);
    if (num_rows == 0 || cols == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q6k || !qs || !d) return LARQL_E_ARG;
    std::vector<uint8_t> packed(q8k_bytes(cols), 0);  // [codes | scales | sums]: this kernel forms its own sums of codes
    memcpy(packed.data(), qs, cols);
    memcpy(packed.data() + cols, d, (cols / 256) * 4);
    return host_matvec_multi(c, KIND_Q6K_Q8K, 1, &q6k, &need, nullptr, nullptr, &num_rows, cols, (const float *)packed.data(), packed.size(), &out);
}

int larql_hip_q4k_dual_matvec(larql_hip_ctx *c, const uint8_t *a, size_t a_len, const uint8_t *b, size_t b_len,
                              const float *x, size_t x_len, size_t num_rows, size_t hidden, float *out_a, float *out_b,
                              size_t out_len) {
    if (!c || ((!out_a || !out_b) && out_len)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (!q4k_shape_ok(out_len, num_rows, x_len, hidden, a_len) || !q4k_shape_ok(out_len, num_rows, x_len, hidden, b_len))
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_dual_matvec: refused operands");
    if (num_rows == 0 || hidden == 0) {
        for (size_t i = 0; i < out_len; i++) { out_a[i] = 0.0f; out_b[i] = 0.0f; }
        return LARQL_OK;
    }
    if (!a || !b || !x) return LARQL_E_ARG;
    const size_t need = (hidden / 256) * 144 * num_rows;
    const uint8_t *w[2] = {a, b};
    const size_t wl[2] = {need, need}, rows[2] = {num_rows, num_rows};
    float *outs[2] = {out_a, out_b};
    return host_matvec_multi(c, KIND_Q4K, 2, w, wl, nullptr, nullptr, rows, hidden, x, x_len * 4, outs);
}

int larql_hip_q4k_matmul(larql_hip_ctx *c, const uint8_t *q4k, size_t q4k_len, const float *x, size_t x_len,
                         size_t num_rows, size_t hidden, size_t seq_len, float *out, size_t out_len) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (out_len != seq_len * num_rows || x_len != seq_len * hidden || (!out && out_len))
        return fail(c, LARQL_REFUSED_SHAPE, "q4k_matmul: out/x lengths do not match [seq, rows] / [seq, hidden]");
    // a zero dimension zero-fills whatever `out` there is (kquant_matmul_into, q4_common/matmul.rs:89-92): hidden == 0
    // with rows and positions leaves seq * rows zeros, the other two leave an empty result
    if (num_rows == 0 || hidden == 0 || seq_len == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return LARQL_OK; }
    if (hidden % 256 != 0 || q4k_len < num_rows * (hidden / 256) * 144) {
        for (size_t i = 0; i < out_len; i++) out[i] = 0.0f;  // the CPU kernel zero-fills on a bad shape
        return LARQL_OK;
    }
    if (!q4k || !x) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    const size_t need = num_rows * (hidden / 256) * 144;
    const uint8_t *dw = nullptr;
    int rc = resolve_weights(c, q4k, need, c->w[0], &dw);
    if (rc) return rc;
    rc = upload(c, c->x, x, x_len * 4);
    if (rc) return rc;
    rc = ensure(c, c->out, out_len * 4 + 64);
    if (rc) return rc;
    Submission sub(c);
    if (seq_len >= 16 && num_rows <= 0xFFFFFFFFull && seq_len <= 0xFFFFFFFFull) {
        // prefill shape: MFMA GEMM on integer weights.  The f32 activations become two f16 terms (per-token
        // scale), so the result keeps ~22 significant bits of x; the second pass is skipped when no lo term exists.
        const size_t sx_len = seq_len * (hidden / 32) * 2;
        rc = ensure(c, c->misc, x_len * 4 + sx_len * 2 + seq_len * 4 + 256);
        if (rc) return rc;
        uint16_t *xh = (uint16_t *)c->misc.p, *xl = xh + x_len, *sx = xl + x_len;
        float *ts = (float *)(((uintptr_t)(sx + sx_len) + 15) & ~(uintptr_t)15);
        HIPCHECK(c, hipMemsetAsync(c->nan_flag + 1, 0, sizeof(int), c->stream));
        HIPCHECK(c, q4k_gemm_prep_launch(c->stream, c->x.p, 0, (uint32_t)hidden, (uint32_t)seq_len, xh, xl, sx, ts, c->nan_flag + 1, nullptr, 0, nullptr));
        int any_lo = 0;
        HIPCHECK(c, hipMemcpyAsync(&any_lo, c->nan_flag + 1, sizeof(int), hipMemcpyDeviceToHost, c->stream));
        HIPCHECK(c, wait_stream(c));
        HIPCHECK(c, hipMemsetAsync(c->nan_flag + 1, 0, sizeof(int), c->stream));
        const uint32_t splits = q4k_gemm_splits((uint32_t)num_rows, (uint32_t)hidden, (uint32_t)seq_len, (uint32_t)c->cu_count);
        float *partial = nullptr;
        if (splits > 1) { rc = ensure(c, c->scores, (size_t)splits * seq_len * num_rows * 4 + 64); if (rc) return rc; partial = (float *)c->scores.p; }
        HIPCHECK(c, q4k_gemm_f16_launch(c->stream, dw, xh, sx, nullptr, ts, (float *)c->out.p, (uint32_t)num_rows, (uint32_t)hidden, (uint32_t)seq_len, 1, 0,
                                        splits, partial));
        if (any_lo)
            HIPCHECK(c, q4k_gemm_f16_launch(c->stream, dw, xl, sx, nullptr, ts, (float *)c->out.p, (uint32_t)num_rows, (uint32_t)hidden, (uint32_t)seq_len, 0, 1,
                                            splits, partial));
    } else {
        std::vector<GemvJob> jobs;
        for (size_t s = 0; s < seq_len; s++)
            jobs.push_back(make_job(KIND_Q4K, dw, nullptr, (const float *)c->x.p + s * hidden, (float *)c->out.p + s * num_rows,
                                    num_rows, hidden));
        rc = enqueue_jobs(c, jobs);
        if (rc) { (void)hipStreamSynchronize(c->stream); return rc; }
    }
    HIPCHECK(c, hipMemcpyAsync(out, c->out.p, out_len * 4, hipMemcpyDeviceToHost, c->stream));
    return sub.finish();
}

// Where a host-tier top-K leaves its hits: idx [batch*k] u32 | val [batch*k] f32 | count [batch] u32.  Small results
// are written by the kernel straight into page-locked host memory (the NaN flag follows them there by one 4-byte copy
// queued behind the kernel), so the call waits for the stream once and copies nothing back; large ones stay in device
// memory and are copied.
struct TopkArea {
    uint32_t *idx;
    float *val;
    uint32_t *cnt;
    bool direct;
};

static int topk_area(larql_hip_ctx *c, size_t batch, size_t k, TopkArea &a) {
    const size_t bytes = batch * (k * 8 + 4);
    a.direct = bytes <= kPinSmall && ensure_pinned(c, c->pin_out, kPinSmall + 64) == LARQL_OK;
    if (!a.direct) { int rc = ensure(c, c->misc, bytes + 64); if (rc) return rc; }
    a.idx = (uint32_t *)(a.direct ? c->pin_out.dev : c->misc.p);
    a.val = (float *)(a.idx + batch * k);
    a.cnt = (uint32_t *)(a.val + batch * k);
    return LARQL_OK;
}

// queued behind the top-K launch, before the call waits for the stream
static int topk_queue_flag(larql_hip_ctx *c, const TopkArea &a) {
    if (a.direct) HIPCHECK(c, hipMemcpyAsync((uint8_t *)c->pin_out.host + kPinSmall, c->nan_flag + 1, sizeof(int), hipMemcpyDeviceToHost, c->stream));
    return LARQL_OK;
}

// after the stream has been waited for
static int topk_collect(larql_hip_ctx *c, const TopkArea &a, size_t batch, size_t k, uint32_t *idx_out, float *score_out, size_t *n_out,
                        bool check_nan) {
    int nan = 0;
    if (a.direct) {
        const uint8_t *h = (const uint8_t *)c->pin_out.host;
        memcpy(idx_out, h, batch * k * 4);
        memcpy(score_out, h + batch * k * 4, batch * k * 4);
        const uint32_t *cnt = (const uint32_t *)(h + batch * k * 8);
        for (size_t b = 0; b < batch; b++) n_out[b] = cnt[b];
        memcpy(&nan, h + kPinSmall, sizeof(int));
    } else {
        std::vector<uint32_t> cnt(batch);
        HIPCHECK(c, hipMemcpyAsync(idx_out, a.idx, batch * k * 4, hipMemcpyDeviceToHost, c->stream));
        HIPCHECK(c, hipMemcpyAsync(score_out, a.val, batch * k * 4, hipMemcpyDeviceToHost, c->stream));
        HIPCHECK(c, hipMemcpyAsync(cnt.data(), a.cnt, batch * 4, hipMemcpyDeviceToHost, c->stream));
        HIPCHECK(c, hipMemcpyAsync(&nan, c->nan_flag + 1, sizeof(int), hipMemcpyDeviceToHost, c->stream));
        HIPCHECK(c, wait_stream(c));
        for (size_t b = 0; b < batch; b++) n_out[b] = cnt[b];
    }
    if (check_nan && nan) return fail(c, LARQL_E_NAN, "top-K: NaN score");
    return LARQL_OK;
}

// matvec + top-K by value with the scores kept on the device (lm_head KNN: lm_head/knn.rs:126-185)
static int host_matvec_topk(larql_hip_ctx *c, int kind, const uint8_t *w, size_t need, const float *x, size_t x_len, size_t num_rows,
                            size_t hidden, size_t top_k, uint32_t *idx_out, float *score_out, size_t *n_out) {
    HIPCHECK(c, hipSetDevice(c->device));
    const uint8_t *dw = nullptr;
    int rc = resolve_weights(c, w, need, c->w[0], &dw);
    if (rc) return rc;
    rc = upload(c, c->x, x, x_len * 4);
    if (rc) return rc;
    rc = ensure(c, c->scores, num_rows * 4 + 64);
    if (rc) return rc;
    TopkArea hits;
    rc = topk_area(c, 1, top_k, hits);
    if (rc) return rc;
    std::vector<GemvJob> jobs{make_job(kind, dw, nullptr, c->x.p, (float *)c->scores.p, num_rows, hidden)};
    Submission sub(c);
    rc = enqueue_jobs(c, jobs);
    if (rc) { (void)wait_stream(c); return rc; }
    HIPCHECK(c, topk_launch(c->stream, (const float *)c->scores.p, 1, (uint32_t)num_rows, (uint32_t)top_k, false, hits.idx, hits.val,
                            hits.cnt, c->nan_flag + 1, nullptr, 0));
    rc = topk_queue_flag(c, hits);
    if (rc) return rc;
    rc = sub.finish();
    if (rc) return rc;
    return topk_collect(c, hits, 1, top_k, idx_out, score_out, n_out, false);
}

int larql_hip_q4k_matvec_topk(larql_hip_ctx *c, const uint8_t *q4k, size_t q4k_len, const float *x, size_t x_len,
                              size_t num_rows, size_t hidden, size_t top_k, uint32_t *idx_out, float *score_out,
                              size_t *n_out) {
    if (!c || !n_out) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    // refusals of the GPU peer (larql-compute-metal/src/trait_impl/quant_matvec.rs:210-215), with this
    // kernel's own capacity (kTopkMaxK) in place of K_TOPK
    if (top_k == 0 || top_k > kTopkMaxK || num_rows == 0 || x_len != hidden) return fail(c, LARQL_UNSUPPORTED, "q4k_matvec_topk: refused");
    if (!q4k_shape_ok(num_rows, num_rows, x_len, hidden, q4k_len)) return fail(c, LARQL_REFUSED_SHAPE, "q4k_matvec_topk: refused operands");
    if (num_rows > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "q4k_matvec_topk: too many rows");
    if (!q4k || !x || !idx_out || !score_out) return LARQL_E_ARG;
    return host_matvec_topk(c, KIND_Q4K, q4k, (hidden / 256) * 144 * num_rows, x, x_len, num_rows, hidden, top_k, idx_out, score_out, n_out);
}

int larql_hip_q8_0_gemv_topk(larql_hip_ctx *c, const uint8_t *blocks, size_t blocks_len, const float *x, size_t x_len, size_t n, size_t k,
                             size_t top_k, uint32_t *idx_out, float *score_out, size_t *n_out) {
    if (!c || !n_out) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (k == 0 || k % 32 != 0 || x_len != k || blocks_len != n * (k / 32) * 34)
        return fail(c, LARQL_REFUSED_SHAPE, "q8_0_gemv_topk: geometry does not describe this pack");
    if (top_k == 0 || top_k > kTopkMaxK || n == 0 || n > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "q8_0_gemv_topk: refused");
    if (!blocks || !x || !idx_out || !score_out) return LARQL_E_ARG;
    return host_matvec_topk(c, KIND_Q8_0, blocks, blocks_len, x, x_len, n, k, top_k, idx_out, score_out, n_out);
}

int larql_hip_q4_matvec(larql_hip_ctx *c, const uint8_t *q4, size_t q4_len, const int8_t *q8_x, size_t q8_len,
                        const float *q8_scales, size_t n_scales, size_t num_rows, size_t hidden, float *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    // the CPU path asserts these (cpu/ops/q4_matvec.rs:37-62); a refusal stands in for the panic
    if (hidden % 32 != 0 || q4_len != num_rows * (hidden / 32) * 18 || q8_len != hidden || n_scales != hidden / 32)
        return fail(c, LARQL_REFUSED_SHAPE, "q4_matvec: refused operands");
    if (num_rows == 0) return LARQL_OK;
    if (hidden == 0) { for (size_t i = 0; i < num_rows; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!q4 || !q8_x || !q8_scales || !out) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    const uint8_t *dw = nullptr;
    int rc = resolve_weights(c, q4, q4_len, c->w[0], &dw);
    if (rc) return rc;
    rc = upload(c, c->q8, q8_x, q8_len);
    if (rc) return rc;
    rc = upload(c, c->q8s, q8_scales, n_scales * 4);
    if (rc) return rc;
    ResultArea res;
    rc = result_area(c, num_rows * 4, res);
    if (rc) return rc;
    std::vector<GemvJob> jobs{make_job(KIND_Q4_0, dw, c->q8s.p, c->q8.p, res.dev, num_rows, hidden)};
    Submission sub(c);
    rc = enqueue_jobs(c, jobs);
    if (rc) { (void)wait_stream(c); return rc; }
    return finish_with_result(c, sub, res, out, num_rows * 4);
}

int larql_hip_q8_0_gemv(larql_hip_ctx *c, const uint8_t *blocks, size_t blocks_len, const float *x, size_t x_len, size_t n,
                        size_t k, float *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (k == 0 || k % 32 != 0 || x_len != k || blocks_len != n * (k / 32) * 34)
        return fail(c, LARQL_REFUSED_SHAPE, "q8_0_gemv: geometry does not describe this pack");
    if (n == 0) return LARQL_OK;
    if (!blocks || !x || !out) return LARQL_E_ARG;
    return host_matvec_multi(c, KIND_Q8_0, 1, &blocks, &blocks_len, nullptr, nullptr, &n, k, x, x_len * 4, &out);
}

int larql_hip_quant_matvec(larql_hip_ctx *c, int format, const uint8_t *weights, size_t w_len, const float *x, size_t x_len,
                           size_t num_rows, size_t hidden, float *out) {
    if (!c) return LARQL_E_ARG;
    switch (format) {
        case LARQL_FMT_Q4_K: case LARQL_FMT_Q4_KF:
            return larql_hip_q4k_matvec(c, weights, w_len, x, x_len, num_rows, hidden, out, num_rows);
        case LARQL_FMT_Q6_K:
            return larql_hip_q6k_matvec(c, weights, w_len, x, x_len, num_rows, hidden, out);
        case LARQL_FMT_Q4_0: {
            std::lock_guard<std::mutex> lk(c->mu);
            if (hidden % 32 != 0 || w_len != num_rows * (hidden / 32) * 18 || x_len != hidden)
                return fail(c, LARQL_REFUSED_SHAPE, "quant_matvec(Q4_0): refused operands");
            if (num_rows == 0) return LARQL_OK;
            if (hidden == 0) { for (size_t i = 0; i < num_rows; i++) out[i] = 0.0f; return LARQL_OK; }
            HIPCHECK(c, hipSetDevice(c->device));
            const uint8_t *dw = nullptr;
            int rc = resolve_weights(c, weights, w_len, c->w[0], &dw);
            if (rc) return rc;
            rc = upload(c, c->x, x, x_len * 4);
            if (rc) return rc;
            rc = ensure(c, c->q8, hidden + 64); if (rc) return rc;
            rc = ensure(c, c->q8s, (hidden / 32) * 4 + 64); if (rc) return rc;
            ResultArea res;
            rc = result_area(c, num_rows * 4, res); if (rc) return rc;
            Submission sub(c);
            HIPCHECK(c, quantize_to_q8_launch(c->stream, (const float *)c->x.p, hidden, (int8_t *)c->q8.p, (float *)c->q8s.p));
            std::vector<GemvJob> jobs{make_job(KIND_Q4_0, dw, c->q8s.p, c->q8.p, res.dev, num_rows, hidden)};
            rc = enqueue_jobs(c, jobs);
            if (rc) { (void)wait_stream(c); return rc; }
            return finish_with_result(c, sub, res, out, num_rows * 4);
        }
        default:
            // Q5_K, I2S, MXFP4 (external scales), the trait's own Q8_0 layout and the
            // float formats answer None through this signature (backend/quant_matvec.rs:58-97).
        {
            std::lock_guard<std::mutex> lk(c->mu);
            return fail(c, LARQL_UNSUPPORTED, "quant_matvec: format %d is not served through this entry", format);
        }
    }
}

int larql_hip_quant_matvec_q8_input(larql_hip_ctx *c, int format, const uint8_t *weights, size_t w_len, const int8_t *q8_x, size_t q8_len,
                                    const float *q8_scales, size_t n_scales, size_t num_rows, size_t hidden, float *out) {
    if (!c) return LARQL_E_ARG;
    switch (format) {
        case LARQL_FMT_Q4_0:
            return larql_hip_q4_matvec(c, weights, w_len, q8_x, q8_len, q8_scales, n_scales, num_rows, hidden, out);
        case LARQL_FMT_Q4_K: case LARQL_FMT_Q4_KF: case LARQL_FMT_Q6_K: {
            // f32-input kernels: dequantise_q8 first (quant_matvec.rs:24-39), then the f32 path
            if ((!q8_x && q8_len) || (!q8_scales && n_scales)) return LARQL_E_ARG;
            const size_t n_blocks = q8_len / 32;
            if (n_scales < n_blocks) {
                std::lock_guard<std::mutex> lk(c->mu);
                return fail(c, LARQL_REFUSED_SHAPE, "quant_matvec_q8_input: %zu scales for %zu blocks", n_scales, n_blocks);
            }
            std::vector<float> xf(q8_len);
            for (size_t b = 0; b < n_blocks; b++)
                for (size_t j = 0; j < 32; j++) xf[b * 32 + j] = (float)q8_x[b * 32 + j] * q8_scales[b];
            for (size_t i = n_blocks * 32; i < q8_len; i++) xf[i] = (float)q8_x[i];
            return larql_hip_quant_matvec(c, format, weights, w_len, xf.data(), xf.size(), num_rows, hidden, out);
        }
        default: {
            // the trait's own Q8_0 layout has no kernel here (as on the CPU backend: q8_matvec -> None); Q5_K, I2S, MXFP4
            // and the float formats answer None through this signature (quant_matvec.rs:126-150)
            std::lock_guard<std::mutex> lk(c->mu);
            return fail(c, LARQL_UNSUPPORTED, "quant_matvec_q8_input: format %d is not served through this entry", format);
        }
    }
}

// ---- host tier: dense / MXFP4 gemv ---------------------------------------------------

static int host_dense_gemv(larql_hip_ctx *c, int kind, const void *w, size_t w_len, const float *x, size_t x_len, size_t n,
                           size_t k, float *out, int force) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const size_t need = n * k * dense_elem_bytes(kind);
    if (w_len < need || x_len != k) return fail(c, LARQL_REFUSED_SHAPE, "gemv: refused operands");
    if (!force && 2 * n * k < c->flop_threshold) return fail(c, LARQL_UNSUPPORTED, "gemv: below the flop threshold");
    if (n == 0) return LARQL_OK;
    if (k == 0) { for (size_t i = 0; i < n; i++) out[i] = 0.0f; return LARQL_OK; }
    if (!w || !x || !out) return LARQL_E_ARG;
    const uint8_t *wp = (const uint8_t *)w;
    return host_matvec_multi(c, kind, 1, &wp, &need, nullptr, nullptr, &n, k, x, x_len * 4, &out);
}

int larql_hip_f32_gemv(larql_hip_ctx *c, const float *w, size_t w_len, const float *x, size_t x_len, size_t n, size_t k,
                       float *out, int force) {
    return host_dense_gemv(c, KIND_F32, w, w_len, x, x_len, n, k, out, force);
}
int larql_hip_f16_gemv(larql_hip_ctx *c, const uint8_t *w, size_t w_len, const float *x, size_t x_len, size_t n, size_t k,
                       float *out, int force) {
    return host_dense_gemv(c, KIND_F16, w, w_len, x, x_len, n, k, out, force);
}
int larql_hip_bf16_gemv(larql_hip_ctx *c, const uint8_t *w, size_t w_len, const float *x, size_t x_len, size_t n, size_t k,
                        float *out, int force) {
    return host_dense_gemv(c, KIND_BF16, w, w_len, x, x_len, n, k, out, force);
}

// MatMul::{bf16,f16}_gemv_multi — backend/matmul.rs:151-194: several matrices against one x as one submission (up to
// kHostMats per launch; more are submitted in groups), results bit-identical to the sequential force gemvs.
static int host_dense_gemv_multi(larql_hip_ctx *c, int kind, size_t n_mats, const uint8_t *const *w, const size_t *w_len, const size_t *n,
                                 const size_t *k, const float *x, size_t x_len, float *const *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n_mats && (!w || !w_len || !n || !k || !out)) return LARQL_E_ARG;
    // any one bad matrix refuses the whole batch, before anything is written (larql-compute-metal/src/trait_impl/matmul.rs:97-126)
    for (size_t i = 0; i < n_mats; i++)
        if (k[i] != x_len || w_len[i] < n[i] * k[i] * dense_elem_bytes(kind))
            return fail(c, LARQL_REFUSED_SHAPE, "gemv_multi: matrix %zu refused (k %zu against x.len() %zu, %zu bytes)", i, k[i], x_len, w_len[i]);
    if (n_mats == 0) return LARQL_OK;  // Some(vec![])
    if (x_len == 0) { for (size_t i = 0; i < n_mats; i++) for (size_t r = 0; r < n[i]; r++) out[i][r] = 0.0f; return LARQL_OK; }
    if (!x) return LARQL_E_ARG;
    for (size_t i = 0; i < n_mats; i += kHostMats) {
        const size_t jn = std::min(kHostMats, n_mats - i);
        size_t need[kHostMats];
        for (size_t t = 0; t < jn; t++) need[t] = n[i + t] * x_len * dense_elem_bytes(kind);
        int rc = host_matvec_multi(c, kind, jn, w + i, need, nullptr, nullptr, n + i, x_len, x, x_len * 4, out + i);
        if (rc) return rc;
    }
    return LARQL_OK;
}
int larql_hip_bf16_gemv_multi(larql_hip_ctx *c, size_t n_mats, const uint8_t *const *w, const size_t *w_len, const size_t *n, const size_t *k,
                              const float *x, size_t x_len, float *const *out) {
    return host_dense_gemv_multi(c, KIND_BF16, n_mats, w, w_len, n, k, x, x_len, out);
}
int larql_hip_f16_gemv_multi(larql_hip_ctx *c, size_t n_mats, const uint8_t *const *w, const size_t *w_len, const size_t *n, const size_t *k,
                             const float *x, size_t x_len, float *const *out) {
    return host_dense_gemv_multi(c, KIND_F16, n_mats, w, w_len, n, k, x, x_len, out);
}

int larql_hip_mxfp4_gemv_multi(larql_hip_ctx *c, size_t n_mats, const uint8_t *const *packed, const size_t *packed_len,
                               const uint8_t *const *scales, const size_t *scales_len, const size_t *n, const size_t *k,
                               const float *x, size_t x_len, float *const *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    for (size_t i = 0; i < n_mats; i++) {
        // larql-compute-metal/src/trait_impl/matmul.rs:267-275
        if (k[i] % 32 != 0 || x_len < k[i] || packed_len[i] < n[i] * (k[i] / 32) * 16 || scales_len[i] < n[i] * (k[i] / 32))
            return fail(c, LARQL_REFUSED_SHAPE, "mxfp4_gemv: matrix %zu refused", i);
    }
    if (n_mats == 0) return LARQL_OK;
    HIPCHECK(c, hipSetDevice(c->device));
    // matrices may differ in k: submit in groups of up to 4 with equal k (results do not depend on grouping)
    size_t i = 0;
    while (i < n_mats) {
        size_t jn = 1;
        while (i + jn < n_mats && jn < 4 && k[i + jn] == k[i]) jn++;
        const uint8_t *w[4], *a[4]; size_t wl[4], al[4], rows[4]; float *outs[4];
        for (size_t t = 0; t < jn; t++) {
            w[t] = packed[i + t]; a[t] = scales[i + t]; rows[t] = n[i + t]; outs[t] = out[i + t];
            wl[t] = n[i + t] * (k[i] / 32) * 16; al[t] = n[i + t] * (k[i] / 32);
        }
        if (k[i] == 0) { for (size_t t = 0; t < jn; t++) for (size_t r = 0; r < rows[t]; r++) outs[t][r] = 0.0f; }
        else {
            int rc = host_matvec_multi(c, KIND_MXFP4, jn, w, wl, a, al, rows, k[i], x, k[i] * 4, outs);
            if (rc) return rc;
        }
        i += jn;
    }
    return LARQL_OK;
}

int larql_hip_mxfp4_gemv(larql_hip_ctx *c, const uint8_t *packed, size_t packed_len, const uint8_t *scales, size_t scales_len,
                         const float *x, size_t x_len, size_t n, size_t k, float *out) {
    // mxfp4_gemv = one-element multi (larql-compute-metal/src/trait_impl/matmul.rs:245-255)
    return larql_hip_mxfp4_gemv_multi(c, 1, &packed, &packed_len, &scales, &scales_len, &n, &k, x, x_len, &out);
}

// ---- gate-KNN ----------------------------------------------------------------------------

static size_t format_row_bytes(int kind, size_t k) {
    switch (kind) {
        case KIND_Q4K: return (k / 256) * 144;
        case KIND_Q4_0: return (k / 32) * 18;
        case KIND_BF16: case KIND_F16: return k * 2;
        case KIND_F32: return k * 4;
        default: return 0;
    }
}

// One gate matrix against `batch` residual positions (x: [batch, hidden], scores: [batch, n]): jobs that
// carry as many positions as the kernels take at once, so the matrix is read once per group.
static void push_gate_jobs(std::vector<GemvJob> &jobs, int kind, const void *gate, const float *x, size_t batch, size_t n,
                           size_t hidden, float *scores) {
    const size_t cap = gemv_batch_capacity(kind, hidden);
    for (size_t b = 0; b < batch;) {
        const size_t take = std::min(cap, batch - b);
        GemvJob j = make_job(kind, gate, nullptr, x + b * hidden, scores + b * n, n, hidden);
        if (take >= 2) { j.batch = (uint32_t)take; j.x_stride = hidden; j.out_stride = n; }
        jobs.push_back(j);
        b += take;
    }
}

// scores[batch, n] on the device for resident gate + x (x: [batch, hidden] f32)
static int dev_gate_scores(larql_hip_ctx *c, int kind, const void *gate, const float *x, size_t batch, size_t n, size_t hidden,
                           float *scores) {
    std::vector<GemvJob> jobs;
    if (kind == KIND_Q4_0) {
        // gate_knn_q4 (dispatch.rs:354-382): quantize_to_q8 per residual, then the Q4_0 x Q8 kernel
        int rc = ensure(c, c->q8, batch * hidden + 64); if (rc) return rc;
        rc = ensure(c, c->q8s, batch * (hidden / 32) * 4 + 64); if (rc) return rc;
        HIPCHECK(c, quantize_to_q8_launch(c->stream, x, batch * hidden, (int8_t *)c->q8.p, (float *)c->q8s.p));
        for (size_t b = 0; b < batch; b++)
            jobs.push_back(make_job(kind, gate, (const float *)c->q8s.p + b * (hidden / 32), (const int8_t *)c->q8.p + b * hidden,
                                    scores + b * n, n, hidden));
    } else {
        push_gate_jobs(jobs, kind, gate, x, batch, n, hidden, scores);
    }
    return enqueue_jobs(c, jobs);
}

static int gate_shape_check(larql_hip_ctx *c, int kind, size_t gate_len, size_t n, size_t hidden) {
    if (kind != KIND_Q4K && kind != KIND_Q4_0 && kind != KIND_BF16 && kind != KIND_F16 && kind != KIND_F32)
        return fail(c, LARQL_UNSUPPORTED, "gate-KNN: unsupported gate format");
    if (kind == KIND_Q4K && hidden % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "gate-KNN: hidden not a multiple of 256");
    if (kind == KIND_Q4_0 && hidden % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "gate-KNN: hidden not a multiple of 32");
    if (gate_len < n * format_row_bytes(kind, hidden)) return fail(c, LARQL_REFUSED_SHAPE, "gate-KNN: gate matrix too short");
    return LARQL_OK;
}

int larql_hip_gate_scores(larql_hip_ctx *c, int format, const uint8_t *gate, size_t gate_len, const float *x, size_t batch,
                          size_t n, size_t hidden, float *scores_out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const int kind = kind_of_format(format);
    int rc = gate_shape_check(c, kind, gate_len, n, hidden);
    if (rc) return rc;
    if (batch == 0 || n == 0) return LARQL_OK;
    if (hidden == 0) { for (size_t i = 0; i < batch * n; i++) scores_out[i] = 0.0f; return LARQL_OK; }
    if (!gate || !x || !scores_out) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    const uint8_t *dg = nullptr;
    rc = resolve_weights(c, gate, n * format_row_bytes(kind, hidden), c->w[0], &dg); if (rc) return rc;
    rc = upload(c, c->x, x, batch * hidden * 4); if (rc) return rc;
    rc = ensure(c, c->scores, batch * n * 4 + 64); if (rc) return rc;
    Submission sub(c);
    rc = dev_gate_scores(c, kind, dg, (const float *)c->x.p, batch, n, hidden, (float *)c->scores.p);
    if (rc) { (void)hipStreamSynchronize(c->stream); return rc; }
    HIPCHECK(c, hipMemcpyAsync(scores_out, c->scores.p, batch * n * 4, hipMemcpyDeviceToHost, c->stream));
    return sub.finish();
}

int larql_hip_gate_knn(larql_hip_ctx *c, int format, const uint8_t *gate, size_t gate_len, const float *x, size_t batch,
                       size_t n, size_t hidden, size_t top_k, uint32_t *idx_out, float *score_out, size_t *n_out) {
    if (!c || (batch && !n_out)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const int kind = kind_of_format(format);
    int rc = gate_shape_check(c, kind, gate_len, n, hidden);
    if (rc) return rc;
    for (size_t b = 0; b < batch; b++) n_out[b] = 0;
    if (batch == 0 || n == 0 || top_k == 0) return LARQL_OK;  // top_k_by_abs: K==0 or no scores -> empty
    if (top_k > kTopkMaxK) return fail(c, LARQL_UNSUPPORTED, "gate-KNN: top_k above %u is not served by this kernel", kTopkMaxK);
    if (n > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "gate-KNN: too many features");
    if (hidden == 0) return fail(c, LARQL_UNSUPPORTED, "gate-KNN: hidden == 0");
    if (!gate || !x || !idx_out || !score_out) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    const uint8_t *dg = nullptr;
    rc = resolve_weights(c, gate, n * format_row_bytes(kind, hidden), c->w[0], &dg); if (rc) return rc;
    rc = upload(c, c->x, x, batch * hidden * 4); if (rc) return rc;
    rc = ensure(c, c->scores, batch * n * 4 + 64); if (rc) return rc;
    TopkArea hits;
    rc = topk_area(c, batch, top_k, hits); if (rc) return rc;
    HIPCHECK(c, hipMemsetAsync(c->nan_flag + 1, 0, sizeof(int), c->stream));
    Submission sub(c);
    rc = dev_gate_scores(c, kind, dg, (const float *)c->x.p, batch, n, hidden, (float *)c->scores.p);
    if (rc) { (void)wait_stream(c); return rc; }
    HIPCHECK(c, topk_launch(c->stream, (const float *)c->scores.p, (uint32_t)batch, (uint32_t)n, (uint32_t)top_k, true, hits.idx,
                            hits.val, hits.cnt, c->nan_flag + 1, nullptr, 0));
    rc = topk_queue_flag(c, hits); if (rc) return rc;
    rc = sub.finish();
    if (rc) return rc;
    return topk_collect(c, hits, batch, top_k, idx_out, score_out, n_out, true);
}

// ---- device tier ----------------------------------------------------------------------------

int larql_hip_debug_alloc_events(larql_hip_ctx *c, uint64_t *out) {
    if (!c || !out) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    *out = c->alloc_events;
    return LARQL_OK;
}

int larql_hip_malloc(larql_hip_ctx *c, void **dptr, size_t bytes) {
    if (!c || !dptr) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    c->alloc_events++;
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipMalloc(dptr, bytes ? bytes : 1));
    return LARQL_OK;
}
int larql_hip_free(larql_hip_ctx *c, void *dptr) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, wait_stream(c));
    HIPCHECK(c, hipFree(dptr));
    return LARQL_OK;
}
int larql_hip_memcpy_h2d(larql_hip_ctx *c, void *dst, const void *src, size_t bytes) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, c->stream));
    HIPCHECK(c, wait_stream(c));
    return LARQL_OK;
}
int larql_hip_memcpy_d2h(larql_hip_ctx *c, void *dst, const void *src, size_t bytes) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c->stream));
    HIPCHECK(c, wait_stream(c));
    return LARQL_OK;
}
int larql_hip_memset(larql_hip_ctx *c, void *dst, int value, size_t bytes) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipMemsetAsync(dst, value, bytes, c->stream));
    return LARQL_OK;
}
int larql_hip_synchronize(larql_hip_ctx *c) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, wait_stream(c));
    return LARQL_OK;
}
int larql_hip_event_create(larql_hip_ctx *c, void **event) {
    if (!c || !event) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    hipEvent_t e;
    HIPCHECK(c, hipEventCreate(&e));
    *event = (void *)e;
    return LARQL_OK;
}
int larql_hip_event_record(larql_hip_ctx *c, void *event) {
    if (!c || !event) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipEventRecord((hipEvent_t)event, c->stream));
    return LARQL_OK;
}
int larql_hip_event_elapsed_ms(larql_hip_ctx *c, void *start, void *stop, float *ms) {
    if (!c || !start || !stop || !ms) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipEventSynchronize((hipEvent_t)stop));
    HIPCHECK(c, hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return LARQL_OK;
}
int larql_hip_event_destroy(larql_hip_ctx *c, void *event) {
    if (!c || !event) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipEventDestroy((hipEvent_t)event));
    return LARQL_OK;
}

static int dev_job_from_public(larql_hip_ctx *c, const larql_hip_matvec_job &p, std::vector<GemvJob> &jobs) {
    const int kind = kind_of_format(p.format);
    if (kind < 0) return fail(c, LARQL_UNSUPPORTED, "matvec: format %d has no kernel", p.format);
    if (kind == KIND_MXFP4 && !p.aux) return fail(c, LARQL_E_ARG, "matvec: MXFP4 needs the scale stream");
    if (kind == KIND_Q4_0) return fail(c, LARQL_UNSUPPORTED, "matvec batch: Q4_0 goes through larql_hip_dev_matvec");
    if ((kind == KIND_Q4K || kind == KIND_Q6K || kind == KIND_Q4K_Q8K || kind == KIND_Q6K_Q8K) && p.k % 256 != 0)
        return fail(c, LARQL_REFUSED_SHAPE, "matvec: k not a multiple of 256");
    if (kind == KIND_Q4K_Q8K && p.k / 256 > 40) return fail(c, LARQL_UNSUPPORTED, "matvec: Q4_K x Q8_K rows longer than 10240 have no kernel");
    if (p.k % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "matvec: k not a multiple of 32");
    jobs.push_back(make_job(kind, p.w, p.aux, p.x, p.out, p.rows, p.k));
    return LARQL_OK;
}

int larql_hip_dev_matvec_batch(larql_hip_ctx *c, const larql_hip_matvec_job *pj, size_t n_jobs) {
    if (!c || (!pj && n_jobs)) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    std::vector<GemvJob> jobs;
    for (size_t i = 0; i < n_jobs; i++) {
        int rc = dev_job_from_public(c, pj[i], jobs);
        if (rc) return rc;
    }
    return enqueue_jobs(c, jobs);
}

struct larql_hip_plan {
    std::vector<PreparedLaunch> launches;
};

int larql_hip_plan_create(larql_hip_ctx *c, const larql_hip_matvec_job *pj, size_t n_jobs, larql_hip_plan **out) {
    if (!c || !out || (!pj && n_jobs)) return LARQL_E_ARG;
    *out = nullptr;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    std::vector<GemvJob> jobs;
    for (size_t i = 0; i < n_jobs; i++) {
        int rc = dev_job_from_public(c, pj[i], jobs);
        if (rc) return rc;
    }
    int rc = check_jobs(c, jobs);
    if (rc) return rc;
    larql_hip_plan *plan = new larql_hip_plan();
    for (std::vector<GemvJob> &live : group_by_kind(jobs)) {
        PreparedLaunch P;
        if (live.size() > (size_t)kInlineJobs) {
            if (hipMalloc(&P.table, table_bytes_for(live.size())) != hipSuccess) {
                for (PreparedLaunch &q : plan->launches) if (q.table) (void)hipFree(q.table);
                delete plan;
                return fail(c, LARQL_E_DEVICE, "plan: out of device memory");
            }
        }
        rc = prepare_same_kind(c, live.data(), live.size(), P.table, P);
        if (rc) {
            if (P.table) (void)hipFree(P.table);
            for (PreparedLaunch &q : plan->launches) if (q.table) (void)hipFree(q.table);
            delete plan;
            return rc;
        }
        plan->launches.push_back(P);
    }
    *out = plan;
    return LARQL_OK;
}

int larql_hip_plan_run(larql_hip_ctx *c, larql_hip_plan *plan) {
    if (!c || !plan) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    for (const PreparedLaunch &P : plan->launches) HIPCHECK(c, gemv_launch(c->stream, P.kind, P.L, P.threads, P.grid, P.lds));
    return LARQL_OK;
}

int larql_hip_plan_launch_count(const larql_hip_plan *plan) { return plan ? (int)plan->launches.size() : 0; }

struct larql_hip_sequence {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int launches = 0;
};

int larql_hip_sequence_create(larql_hip_ctx *c, larql_hip_plan *const *plans, size_t n_plans, larql_hip_sequence **out) {
    if (!c || !out || (!plans && n_plans)) return LARQL_E_ARG;
    *out = nullptr;
    for (size_t i = 0; i < n_plans; i++)
        if (!plans[i]) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    // once eagerly: whatever a kernel's first launch sets up (its LDS limit) happens outside the recording
    for (size_t i = 0; i < n_plans; i++)
        for (const PreparedLaunch &P : plans[i]->launches) HIPCHECK(c, gemv_launch(c->stream, P.kind, P.L, P.threads, P.grid, P.lds));
    HIPCHECK(c, wait_stream(c));
    larql_hip_sequence *seq = new larql_hip_sequence();
    hipError_t e = hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal);
    if (e == hipSuccess) {
        for (size_t i = 0; i < n_plans && e == hipSuccess; i++)
            for (const PreparedLaunch &P : plans[i]->launches) {
                e = gemv_launch(c->stream, P.kind, P.L, P.threads, P.grid, P.lds);
                if (e != hipSuccess) break;
                seq->launches++;
            }
        hipGraph_t g = nullptr;
        const hipError_t e2 = hipStreamEndCapture(c->stream, &g);  // (always ends the recording, also after a failed launch)
        seq->graph = g;
        if (e == hipSuccess) e = e2;
    }
    if (e == hipSuccess) e = hipGraphInstantiate(&seq->exec, seq->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        if (seq->exec) (void)hipGraphExecDestroy(seq->exec);
        if (seq->graph) (void)hipGraphDestroy(seq->graph);
        delete seq;
        return fail(c, LARQL_E_DEVICE, "sequence: %s", hipGetErrorString(e));
    }
    *out = seq;
    return LARQL_OK;
}

int larql_hip_sequence_run(larql_hip_ctx *c, larql_hip_sequence *seq) {
    if (!c || !seq) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, hipGraphLaunch(seq->exec, c->stream));
    return LARQL_OK;
}

int larql_hip_sequence_launch_count(const larql_hip_sequence *seq) { return seq ? seq->launches : 0; }

void larql_hip_sequence_destroy(larql_hip_ctx *c, larql_hip_sequence *seq) {
    if (!seq) return;
    if (c) { (void)hipSetDevice(c->device); (void)hipStreamSynchronize(c->stream); }
    if (seq->exec) (void)hipGraphExecDestroy(seq->exec);
    if (seq->graph) (void)hipGraphDestroy(seq->graph);
    delete seq;
}

void larql_hip_plan_destroy(larql_hip_ctx *c, larql_hip_plan *plan) {
    if (!plan) return;
    if (c) { (void)hipSetDevice(c->device); (void)hipStreamSynchronize(c->stream); }
    for (PreparedLaunch &P : plan->launches) if (P.table) (void)hipFree(P.table);
    delete plan;
}

int larql_hip_dev_matvec(larql_hip_ctx *c, int format, const void *w, const void *aux, const float *x, size_t rows, size_t k,
                         float *out) {
    if (!c) return LARQL_E_ARG;
    if (format == LARQL_FMT_Q4_0) {
        std::lock_guard<std::mutex> lk(c->mu);
        HIPCHECK(c, hipSetDevice(c->device));
        if (k % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "matvec: k not a multiple of 32");
        int rc = ensure(c, c->q8, k + 64); if (rc) return rc;
        rc = ensure(c, c->q8s, (k / 32) * 4 + 64); if (rc) return rc;
        HIPCHECK(c, quantize_to_q8_launch(c->stream, x, k, (int8_t *)c->q8.p, (float *)c->q8s.p));
        std::vector<GemvJob> jobs{make_job(KIND_Q4_0, w, c->q8s.p, c->q8.p, out, rows, k)};
        return enqueue_jobs(c, jobs);
    }
    larql_hip_matvec_job j;
    memset(&j, 0, sizeof j);
    j.format = format; j.w = w; j.aux = aux; j.x = x; j.out = out; j.rows = rows; j.k = k;
    return larql_hip_dev_matvec_batch(c, &j, 1);
}

// Clears the NaN flag on the stream (a kernel, not a memset node: see zero_words_kernel).
static int clear_nan_flag(larql_hip_ctx *c) {
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, c->stream, (uint32_t *)c->nan_flag, 1u);
    HIPCHECK(c, hipGetLastError());
    return LARQL_OK;
}

int larql_hip_dev_gate_knn(larql_hip_ctx *c, int format, const void *gate, const float *x, size_t batch, size_t n, size_t hidden,
                           size_t top_k, float *scores_scratch, uint32_t *idx_out, float *score_out, uint32_t *count_out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const int kind = kind_of_format(format);
    int rc = gate_shape_check(c, kind, (size_t)-1, 0, hidden);
    if (rc) return rc;
    if (batch == 0 || n == 0 || top_k == 0) return LARQL_OK;
    if (top_k > kTopkMaxK || n > 0xFFFFFFFFull || hidden == 0) return fail(c, LARQL_UNSUPPORTED, "gate-KNN: unsupported size");
    HIPCHECK(c, hipSetDevice(c->device));
    if (!count_out) { rc = ensure(c, c->misc, batch * 4 + 64); if (rc) return rc; count_out = (uint32_t *)c->misc.p; }
    rc = dev_gate_scores(c, kind, gate, x, batch, n, hidden, scores_scratch);
    if (rc) return rc;
    HIPCHECK(c, topk_launch(c->stream, scores_scratch, (uint32_t)batch, (uint32_t)n, (uint32_t)top_k, true, idx_out, score_out,
                            count_out, c->nan_flag, nullptr, 0));
    return LARQL_OK;
}

int larql_hip_dev_take_nan_flag(larql_hip_ctx *c, int *flag_out) {
    if (!c || !flag_out) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    int v = 0;
    HIPCHECK(c, hipMemcpyAsync(&v, c->nan_flag, sizeof(int), hipMemcpyDeviceToHost, c->stream));
    HIPCHECK(c, wait_stream(c));
    *flag_out = v != 0;
    if (v) { int rc = clear_nan_flag(c); if (rc) return rc; }
    return LARQL_OK;
}

size_t larql_hip_static_scratch_bytes(void) { return kStaticScratchBytes; }

// larql_hip_dev_gate_knn without any allocation: scores, hit counts and the Q8 activation of Q4_0 gates use this
// device's static scratch array; job descriptors travel in the kernel arguments (at most kInlineJobs per launch,
// which batch <= LARQL_HIP_STATIC_MAX_BATCH guarantees); no vector, no staging buffer, no table upload.
int larql_hip_dev_gate_knn_static(larql_hip_ctx *c, int format, const void *gate, const float *x, size_t batch, size_t n,
                                  size_t hidden, size_t top_k, uint32_t *idx_out, float *score_out, uint32_t *count_out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const int kind = kind_of_format(format);
    int rc = gate_shape_check(c, kind, (size_t)-1, 0, hidden);
    if (rc) return rc;
    if (batch == 0 || n == 0 || top_k == 0) return LARQL_OK;
    if (top_k > kTopkMaxK || hidden == 0) return fail(c, LARQL_UNSUPPORTED, "gate-KNN: unsupported size");
    if (batch > LARQL_HIP_STATIC_MAX_BATCH || n > LARQL_HIP_STATIC_MAX_SCORES || batch * n > LARQL_HIP_STATIC_MAX_SCORES)
        return fail(c, LARQL_REFUSED_SHAPE, "gate_knn_static: batch %zu x %zu features exceeds the static scratch (at most %d positions, %d scores)",
                    batch, n, LARQL_HIP_STATIC_MAX_BATCH, LARQL_HIP_STATIC_MAX_SCORES);
    if (kind == KIND_Q4_0 && hidden > LARQL_HIP_STATIC_MAX_HIDDEN)
        return fail(c, LARQL_REFUSED_SHAPE, "gate_knn_static: Q4_0 gates take rows of at most %d elements here", LARQL_HIP_STATIC_MAX_HIDDEN);
    if (!gate || !x || !idx_out || !score_out || !c->static_scratch) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    float *scores = (float *)c->static_scratch;
    uint32_t *counts = (uint32_t *)(c->static_scratch + kStaticScoresBytes);
    int8_t *q8 = (int8_t *)(c->static_scratch + kStaticScoresBytes + kStaticCountsBytes);
    float *q8s = (float *)(c->static_scratch + kStaticScoresBytes + kStaticCountsBytes + kStaticQ8Bytes);
    GemvJob jobs[LARQL_HIP_STATIC_MAX_BATCH];
    size_t n_jobs = 0;
    if (kind == KIND_Q4_0) {
        HIPCHECK(c, quantize_to_q8_launch(c->stream, x, batch * hidden, q8, q8s));
        for (size_t b = 0; b < batch; b++)
            jobs[n_jobs++] = make_job(kind, gate, q8s + b * (hidden / 32), q8 + b * hidden, scores + b * n, n, hidden);
    } else {
        const size_t cap = gemv_batch_capacity(kind, hidden);
        for (size_t b = 0; b < batch;) {
            const size_t take = std::min(cap, batch - b);
            GemvJob j = make_job(kind, gate, nullptr, x + b * hidden, scores + b * n, n, hidden);
            if (take >= 2) { j.batch = (uint32_t)take; j.x_stride = hidden; j.out_stride = n; }
            jobs[n_jobs++] = j;
            b += take;
        }
    }
    for (size_t i = 0; i < n_jobs; i++) {
        if (((uintptr_t)jobs[i].w & 15) || ((uintptr_t)jobs[i].x & 15))
            return fail(c, LARQL_REFUSED_SHAPE, "matvec: weight and activation pointers must be 16-byte aligned");
        jobs[i].kind = gemv_effective_kind(jobs[i]);
    }
    // one launch per kernel the jobs map to (a full group of positions and a single left-over position may differ)
    bool done[LARQL_HIP_STATIC_MAX_BATCH] = {};
    for (size_t i = 0; i < n_jobs; i++) {
        if (done[i]) continue;
        GemvJob live[LARQL_HIP_STATIC_MAX_BATCH];
        size_t n_live = 0;
        for (size_t t = i; t < n_jobs; t++)
            if (!done[t] && jobs[t].kind == jobs[i].kind) { live[n_live++] = jobs[t]; done[t] = true; }
        static_assert(LARQL_HIP_STATIC_MAX_BATCH <= kInlineJobs, "the jobs of a launch must fit the kernel arguments");
        PreparedLaunch P;
        rc = prepare_same_kind(c, live, n_live, nullptr, P);
        if (rc) return rc;
        HIPCHECK(c, gemv_launch(c->stream, P.kind, P.L, P.threads, P.grid, P.lds));
    }
    HIPCHECK(c, topk_launch(c->stream, scores, (uint32_t)batch, (uint32_t)n, (uint32_t)top_k, true, idx_out, score_out,
                            count_out ? count_out : counts, c->nan_flag, nullptr, 0));
    return LARQL_OK;
}

int larql_hip_dev_copy(larql_hip_ctx *c, void *dst, const void *src, size_t bytes) {
    if (!c || !src) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (bytes % 16 != 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return fail(c, LARQL_REFUSED_SHAPE, "copy: 16-byte granularity");
    HIPCHECK(c, hipSetDevice(c->device));
    const uint32_t grid = (uint32_t)c->cu_count * 8u;
    if (dst) HIPCHECK(c, copy_launch(c->stream, src, dst, bytes, grid));
    else { int rc = ensure(c, c->misc, 64); if (rc) return rc; HIPCHECK(c, read_launch(c->stream, src, (uint32_t *)c->misc.p, bytes, grid)); }
    return LARQL_OK;
}

// The GEMM with the rows' exponents either given (row_exp: computed once per matrix) or computed on the way.
static int dev_q4k_gemm(larql_hip_ctx *c, const uint8_t *w, const int32_t *row_exp, const uint16_t *x_bf16, size_t rows, size_t hidden,
                        size_t seq, float *out) {
    if (rows == 0 || seq == 0 || hidden == 0) return LARQL_OK;
    if (hidden % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "q4k_gemm: hidden not a multiple of 256");
    if (rows > 0xFFFFFFFFull || seq > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "q4k_gemm: too large");
    if (!w || !x_bf16 || !out || ((uintptr_t)w & 15) || ((uintptr_t)x_bf16 & 15)) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    // bf16 activations are exact in one f16 term after the per-token scale
    const size_t x_len = seq * hidden, sx_len = seq * (hidden / 32) * 2;
    int rc = ensure(c, c->misc, x_len * 2 + sx_len * 2 + seq * 4 + rows * 4 + 256);
    if (rc) return rc;
    uint16_t *xh = (uint16_t *)c->misc.p, *sx = xh + x_len;
    float *ts = (float *)(((uintptr_t)(sx + sx_len) + 15) & ~(uintptr_t)15);
    // the rows' exponents: the rows' scales ride in the f16 weight operand (1.4e-4 of the CPU value)
    int *rexp = row_exp ? const_cast<int *>((const int *)row_exp) : (int *)(ts + seq);
    HIPCHECK(c, q4k_gemm_prep_launch(c->stream, x_bf16, 1, (uint32_t)hidden, (uint32_t)seq, xh, nullptr, sx, ts, nullptr, row_exp ? nullptr : w,
                                     (uint32_t)rows, row_exp ? nullptr : rexp));
    const uint32_t splits = q4k_gemm_splits((uint32_t)rows, (uint32_t)hidden, (uint32_t)seq, (uint32_t)c->cu_count);
    float *partial = nullptr;
    if (splits > 1) { rc = ensure(c, c->scores, (size_t)splits * seq * rows * 4 + 64); if (rc) return rc; partial = (float *)c->scores.p; }
    HIPCHECK(c, q4k_gemm_f16_launch(c->stream, w, xh, sx, rexp, ts, out, (uint32_t)rows, (uint32_t)hidden, (uint32_t)seq, 1, 0, splits, partial));
    return LARQL_OK;
}

int larql_hip_dev_q4k_gemm(larql_hip_ctx *c, const uint8_t *w, const uint16_t *x_bf16, size_t rows, size_t hidden, size_t seq,
                           float *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    return dev_q4k_gemm(c, w, nullptr, x_bf16, rows, hidden, seq, out);
}

int larql_hip_dev_q4k_gemm_prepared(larql_hip_ctx *c, const uint8_t *w, const int32_t *row_exp, const uint16_t *x_bf16, size_t rows,
                                    size_t hidden, size_t seq, float *out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (!row_exp && rows && seq && hidden) return LARQL_E_ARG;
    return dev_q4k_gemm(c, w, row_exp, x_bf16, rows, hidden, seq, out);
}

int larql_hip_dev_q4k_row_exponents(larql_hip_ctx *c, const uint8_t *w, size_t rows, size_t hidden, int32_t *row_exp) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (rows == 0 || hidden == 0) return LARQL_OK;
    if (hidden % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "q4k_row_exponents: hidden not a multiple of 256");
    if (rows > 0xFFFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "q4k_row_exponents: too large");
    if (!w || !row_exp || ((uintptr_t)w & 15)) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, q4k_gemm_prep_launch(c->stream, nullptr, 1, (uint32_t)hidden, 0, nullptr, nullptr, nullptr, nullptr, nullptr, w, (uint32_t)rows,
                                     (int *)row_exp));
    return LARQL_OK;
}

// ---- device tier: MoE -------------------------------------------------------------------------

int larql_hip_dev_router_select(larql_hip_ctx *c, const float *logits, size_t tokens, size_t n_experts, size_t k, int policy,
                                uint32_t *experts, float *weights) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (k > n_experts) k = n_experts;  // select(): k.min(logits.len())
    if (tokens == 0 || k == 0) return LARQL_OK;
    if (n_experts > kRouterMaxExperts || k > 8) return fail(c, LARQL_UNSUPPORTED, "router_select: at most 256 experts and top-8 on this backend");
    if (!logits || !experts || !weights) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, router_select_launch(c->stream, logits, nullptr, (uint32_t)tokens, (uint32_t)n_experts, (uint32_t)k, policy, experts, weights));
    return LARQL_OK;
}

size_t larql_hip_moe_mxfp4_workspace_bytes(size_t tokens, size_t k, size_t hidden, size_t inter) {
    const size_t slots = tokens * k;
    return (slots * inter * 3 + slots * hidden) * sizeof(float) + 256;
}

// The expert block; with `route_logits` the selection is part of it (written to experts / weights as
// larql_hip_dev_router_select would): inside the first matvec launch for one token, by the selection kernel otherwise.
static int moe_mxfp4_block(larql_hip_ctx *c, const larql_hip_mxfp4_experts *bank, const float *x, size_t tokens, size_t k,
                           uint32_t *experts, float *weights, float *out, void *workspace, size_t workspace_bytes,
                           const float *route_logits, int route_policy) {
    const size_t hidden = bank->hidden, inter = bank->inter;
    if (hidden % 32 != 0 || inter % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "moe_mxfp4: hidden and inter must be multiples of 32");
    if (tokens == 0 || k == 0) return LARQL_OK;
    if (workspace_bytes < larql_hip_moe_mxfp4_workspace_bytes(tokens, k, hidden, inter))
        return fail(c, LARQL_REFUSED_SHAPE, "moe_mxfp4: workspace too small");
    if (!x || !experts || !weights || !out || !workspace) return LARQL_E_ARG;
    if (((uintptr_t)workspace & 15) || ((uintptr_t)x & 15) || ((uintptr_t)bank->gate_packed & 15) || ((uintptr_t)bank->up_packed & 15) ||
        ((uintptr_t)bank->down_packed & 15))
        return fail(c, LARQL_REFUSED_SHAPE, "moe_mxfp4: workspace, activation and packed-weight pointers must be 16-byte aligned");
    if (!bank->gate_packed || !bank->gate_scales || !bank->down_packed || !bank->down_scales ||
        (!bank->gate_up_interleaved && (!bank->up_packed || !bank->up_scales)))
        return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    if (route_logits && tokens == 1 && bank->n_experts > kRouterInLaunchExperts) {
        // more experts than a matvec launch selects over by itself: the selection kernel first, then the block on its choice
        HIPCHECK(c, router_select_launch(c->stream, route_logits, bank->router_bias, 1, (uint32_t)bank->n_experts, (uint32_t)k, route_policy, experts,
                                         weights));
        route_logits = nullptr;
    }
    const size_t slots = tokens * k;
    float *g = (float *)workspace, *u = g + slots * inter, *h = u + slots * inter, *d = h + slots * inter;
    // fused: every expert's gate_up region is one matrix of 2*inter interleaved rows (gate even, up odd), walked in
    // place by one job per slot; its 2*inter results (g0 u0 g1 u1 ...) fill the slot's share of the g and u areas
    const bool fused = bank->gate_up_interleaved != 0;
    const size_t gu_rows = fused ? 2 * inter : inter;
    const uint64_t gu_w_stride = gu_rows * (hidden / 32) * 16, gu_s_stride = gu_rows * (hidden / 32);
    const uint64_t dn_w_stride = hidden * (inter / 32) * 16, dn_s_stride = hidden * (inter / 32);
    // one token: the gate/up launch can select for itself (every wavefront repeats the token's selection, the
    // workgroup that opens the first job writes it out for the launches that follow)
    // Expert biases ride in the jobs: the fused bias row is interleaved (gate bias j at 2j, up bias j at 2j+1) whatever the
    // weight layout, so a fused job adds it element for element and separate gate / up jobs take every second element.
    const auto set_gate_up_bias = [&](GemvJob &jb, int half) {
        if (!bank->gate_up_bias) return;
        jb.bias = bank->gate_up_bias + (fused ? 0 : half);
        jb.bias_step = fused ? 1u : 2u;
        jb.bias_sel_stride = 2 * inter;
    };
    const auto set_down_bias = [&](GemvJob &jb) {
        if (!bank->down_bias) return;
        jb.bias = bank->down_bias; jb.bias_step = 1; jb.bias_sel_stride = hidden;
    };
    if (tokens == 1 && k <= kMoe1MaxK) {
        // One token: a launch for the selected experts' gate / up projections (which selects for itself when it is
        // given the logits) and a launch for their down projections, gated on the way in, folded over the experts,
        // weighted and biased on the way out.
        Moe1Args ga = {}, da = {};
        ga.logits = route_logits; ga.router_bias = bank->router_bias; ga.experts = experts; ga.weights = weights;
        ga.n_experts = (uint32_t)bank->n_experts; ga.k = (uint32_t)k; ga.policy = route_policy;
        ga.n_mats = fused ? 1u : 2u;
        ga.w[0] = (const uint8_t *)bank->gate_packed; ga.aux[0] = (const uint8_t *)bank->gate_scales;
        ga.w[1] = (const uint8_t *)bank->up_packed; ga.aux[1] = (const uint8_t *)bank->up_scales;
        ga.w_stride = gu_w_stride; ga.aux_stride = gu_s_stride;
        if (bank->gate_up_bias) {  // the fused bias row is interleaved (gate bias j at 2j, up bias j at 2j+1) whatever the weight layout
            ga.bias[0] = bank->gate_up_bias; ga.bias[1] = bank->gate_up_bias + 1;
            ga.bias_stride = 2 * inter; ga.bias_step = fused ? 1u : 2u;
        }
        ga.rows = (uint32_t)gu_rows; ga.kdim = (uint32_t)hidden;
        ga.x = x;
        ga.out[0] = g; ga.out[1] = u; ga.out_slot_stride = gu_rows;
        da.experts = experts; da.weights = weights; da.n_experts = (uint32_t)bank->n_experts; da.k = (uint32_t)k; da.n_mats = 1;
        da.w[0] = (const uint8_t *)bank->down_packed; da.aux[0] = (const uint8_t *)bank->down_scales;
        da.w_stride = dn_w_stride; da.aux_stride = dn_s_stride;
        if (bank->down_bias) { da.bias[0] = bank->down_bias; da.bias_stride = hidden; da.bias_step = 1; }
        da.rows = (uint32_t)hidden; da.kdim = (uint32_t)inter;
        da.x = g; da.x_glu = fused ? g : u; da.x_slot_stride = gu_rows;
        da.glu_limit = bank->limit; da.glu_alpha = bank->alpha;
        da.out[0] = out;
        if (fused) {
            // the stages hand the gated activation over as operand terms: 3 x k x kpad bf16 in the workspace's gate / up areas
            // (6 bytes per element where the raw results would take 8)
            const size_t kpad = (inter + 127) / 128 * 128;
            if (3 * k * kpad * sizeof(uint16_t) <= 2 * slots * inter * sizeof(float)) {
                ga.terms = da.terms = (uint16_t *)g;
                ga.terms_kpad = da.terms_kpad = (uint32_t)kpad;
                ga.glu_limit = bank->limit; ga.glu_alpha = bank->alpha;
            }
        }
        uint32_t gt = 0, dt = 0;
        size_t gl = 0, dl = 0;
        if (gu_rows < (1u << 22) && hidden < (1u << 22) && c->cu_count <= 512 && (!route_logits || bank->n_experts <= kRouterInLaunchExperts) && moe1_geometry(ga, &gt, &gl) &&
            moe1_geometry(da, &dt, &dl)) {
            const uint32_t cus = (uint32_t)c->cu_count;
            // a short result is cut into tiles of fewer than 16 rows so that every compute unit gets the same share
            const uint32_t per_wg = (uint32_t)(((hidden + 15) / 16 + cus - 1) / cus);
            da.tile_rows = (uint32_t)std::min<size_t>(16, (hidden + (size_t)cus * per_wg - 1) / ((size_t)cus * per_wg));
            const uint32_t g_units = (uint32_t)(k * ga.n_mats * ((gu_rows + 15) / 16)), d_units = (uint32_t)((hidden + da.tile_rows - 1) / da.tile_rows);
            HIPCHECK(c, moe1_launch(c->stream, ga, false, std::min(cus, g_units), gt, gl));
            HIPCHECK(c, moe1_launch(c->stream, da, true, std::min(cus, d_units), dt, dl));
            return LARQL_OK;
        }
    }
    const bool route_in_launch = route_logits && tokens == 1 &&
        gemv_effective_kind(make_job(KIND_MXFP4, bank->gate_packed, bank->gate_scales, x, g, gu_rows, hidden)) == KIND_MXFP4_MFMA;
    // (the selection kernel, unless the planner below does the selecting itself)
    bool router_pending = route_logits && !route_in_launch;
    // Several tokens: slots that chose the same expert share its weights up to four at a time.  The job lists are built on
    // the device from the router's choice (moe_plan_kernel) into the workspace's spare activation area.
    {
        GemvJob tg = make_job(KIND_MXFP4, bank->gate_packed, bank->gate_scales, x, g, gu_rows, hidden);
        set_gate_up_bias(tg, 0);
        GemvJob tu = fused ? tg : make_job(KIND_MXFP4, bank->up_packed, bank->up_scales, x, u, inter, hidden);
        if (!fused) set_gate_up_bias(tu, 1);
        GemvJob td = make_job(KIND_MXFP4, bank->down_packed, bank->down_scales, g, d, hidden, inter);
        td.x_glu = fused ? g : u; td.glu_limit = bank->limit; td.glu_alpha = bank->alpha;
        set_down_bias(td);
        constexpr uint32_t kFirstMax = 1024;  // workgroups per launch whose first jobs the planner looks up
        const size_t table_bytes = slots * 3 * sizeof(GemvJob) + 64 + 2 * kFirstMax * sizeof(uint32_t);
        const bool mfma = gemv_effective_kind(tg) == KIND_MXFP4_MFMA && gemv_effective_kind(td) == KIND_MXFP4_MFMA;
        if (mfma && tokens > 1 && slots <= 4096 && bank->n_experts <= 1024 && slots * inter * sizeof(float) >= table_bytes) {
            tg.kind = tu.kind = td.kind = KIND_MXFP4_MFMA;
            uint32_t *hdr = (uint32_t *)h;  // {gate/up count, passes, down count, passes}
            GemvJob *gu_table = (GemvJob *)((uint8_t *)h + 64), *dn_table = gu_table + 2 * slots;
            PreparedLaunch Pg, Pd;
            // four tokens per job where the launches' LDS has room for their partial sums, else two
            uint32_t group = 4;
            for (int which = 0; which < 2 && group > 2; which++) {
                GemvJob tj = which == 0 ? tg : td;
                const uint32_t th = gemv_pick_threads(&tj, 1);
                tj.batch = group;
                if (th == 0 || !gemv_job_geometry(tj, th) || gemv_lds_bytes(&tj, 1, th) > 160 * 1024) group = 2;
            }
            for (int which = 0; which < 2; which++) {
                GemvJob &tj = which == 0 ? tg : td;
                PreparedLaunch &P = which == 0 ? Pg : Pd;
                P.kind = KIND_MXFP4_MFMA;
                P.threads = gemv_pick_threads(&tj, 1);
                if (P.threads == 0 || !gemv_job_geometry(tj, P.threads)) return fail(c, LARQL_UNSUPPORTED, "moe_mxfp4: unsupported geometry");
                const uint64_t max_jobs = which == 0 && !fused ? 2 * slots : slots;
                // (the planner's cost per job: at most 1060 units a tile and under 11 more tiles' worth of start-up)
                if (max_jobs * (((uint64_t)tj.rows + 15) / 16 + 11) * 1060 > 0x7FFFFFFFull) return fail(c, LARQL_UNSUPPORTED, "moe_mxfp4: launch too large");
                memset(&P.L, 0, sizeof P.L);
                P.L.table = which == 0 ? gu_table : dn_table;
                P.L.dyn = hdr + 2 * which;
                P.L.pad = gemv_launch_param(&tj, 1);
                tj.batch = group;  // (sizes the partial sums; the planner sets every job's own count)
                P.lds = gemv_lds_bytes(&tj, 1, P.threads);
                P.grid = (uint32_t)((uint64_t)c->cu_count * gemv_wgs_per_cu(P.kind, P.threads, P.lds, (uint32_t)c->wgs_per_cu));
            }
            if (!gemv_job_geometry(tu, Pg.threads)) return fail(c, LARQL_UNSUPPORTED, "moe_mxfp4: unsupported geometry");
            uint32_t *gu_first = nullptr, *dn_first = nullptr;
            if (Pg.grid <= kFirstMax && Pd.grid <= kFirstMax) {
                gu_first = (uint32_t *)(dn_table + slots);
                dn_first = gu_first + kFirstMax;
                Pg.L.wg_first = gu_first;
                Pd.L.wg_first = dn_first;
            }
            HIPCHECK(c, moe_plan_launch(c->stream, router_pending ? route_logits : nullptr, bank->router_bias, route_policy, weights, experts,
                                        (uint32_t)slots, (uint32_t)k, (uint32_t)bank->n_experts, tg, tu, td, gu_w_stride,
                                        gu_s_stride, dn_w_stride, dn_s_stride, (uint32_t)hidden, (uint32_t)inter, fused, group, Pg.grid, Pd.grid, gu_table,
                                        hdr, dn_table, hdr + 2, gu_first, dn_first));
            HIPCHECK(c, gemv_launch(c->stream, Pg.kind, Pg.L, Pg.threads, Pg.grid, Pg.lds));
            HIPCHECK(c, gemv_launch(c->stream, Pd.kind, Pd.L, Pd.threads, Pd.grid, Pd.lds));
            HIPCHECK(c, weighted_sum_launch(c->stream, d, weights, experts, (uint32_t)bank->n_experts, out, (uint32_t)tokens, (uint32_t)k,
                                            (uint32_t)hidden));
            return LARQL_OK;
        }
    }
    if (router_pending)
        HIPCHECK(c, router_select_launch(c->stream, route_logits, bank->router_bias, (uint32_t)tokens, (uint32_t)bank->n_experts, (uint32_t)k,
                                         route_policy, experts, weights));
    std::vector<GemvJob> jobs;
    for (size_t s = 0; s < slots; s++) {
        const size_t t = s / k;
        GemvJob a = make_job(KIND_MXFP4, bank->gate_packed, bank->gate_scales, x + t * hidden, g + s * gu_rows, gu_rows, hidden);
        a.sel = experts + s; a.w_sel_stride = gu_w_stride; a.aux_sel_stride = gu_s_stride; a.sel_count = (uint32_t)bank->n_experts;
        set_gate_up_bias(a, 0);
        if (route_in_launch) {
            a.sel = nullptr;
            a.route_logits = route_logits; a.route_bias = bank->router_bias; a.route_n = (uint32_t)bank->n_experts; a.route_k = (uint32_t)k;
            a.route_rank = (uint32_t)s; a.route_policy = route_policy;
        }
        GemvJob b = a;
        if (route_in_launch && s == 0) { a.route_experts = experts; a.route_weights = weights; }
        jobs.push_back(a);
        if (fused) continue;
        b.w = (const uint8_t *)bank->up_packed; b.aux = (const uint8_t *)bank->up_scales; b.out = u + s * inter; b.rows = inter;
        set_gate_up_bias(b, 1);
        jobs.push_back(b);
    }
    int rc = enqueue_jobs(c, jobs);
    if (rc) return rc;
    // the gated activation is applied by the down projection itself where the matrix-core kernel serves it
    const bool fuse_glu = gemv_effective_kind(make_job(KIND_MXFP4, bank->down_packed, bank->down_scales, g, d, hidden, inter)) != KIND_MXFP4;
    if (!fuse_glu) {
        if (fused) HIPCHECK(c, clamped_glu_interleaved_launch(c->stream, g, h, slots * inter, bank->limit, bank->alpha));
        else HIPCHECK(c, clamped_glu_launch(c->stream, g, u, h, slots * inter, bank->limit, bank->alpha));
    }
    jobs.clear();
    if (fuse_glu && tokens == 1 && k <= 4) {
        // One token: the down projection folds its k experts and the weighted sum — every workgroup walks its output rows
        // through the k experts' matrices, each activation scaled by its routing weight, and writes
        // sum_s w_s * (down_s . act_s + bias_s) itself.  No third launch.
        const size_t gs = fused ? 2 * inter : inter;  // floats of gate/up results per slot
        GemvJob a = make_job(KIND_MXFP4, bank->down_packed, bank->down_scales, g, out, hidden, inter);
        a.x_glu = fused ? g : u; a.glu_limit = bank->limit; a.glu_alpha = bank->alpha;
        a.batch = (uint32_t)k; a.x_stride = gs; a.x_off[0] = (int64_t)(2 * gs); a.x_off[1] = (int64_t)(3 * gs);
        a.sel = experts; a.w_sel_stride = dn_w_stride; a.aux_sel_stride = dn_s_stride; a.sel_count = (uint32_t)bank->n_experts;
        a.combine_w = weights;
        set_down_bias(a);
        jobs.push_back(a);
        return enqueue_jobs(c, jobs);
    }
    for (size_t s = 0; s < slots; s++) {
        const float *gx = fused ? g + s * 2 * inter : g + s * inter;
        GemvJob a = make_job(KIND_MXFP4, bank->down_packed, bank->down_scales, fuse_glu ? gx : h + s * inter, d + s * hidden,
                             hidden, inter);
        if (fuse_glu) { a.x_glu = fused ? gx : u + s * inter; a.glu_limit = bank->limit; a.glu_alpha = bank->alpha; }
        a.sel = experts + s; a.w_sel_stride = dn_w_stride; a.aux_sel_stride = dn_s_stride; a.sel_count = (uint32_t)bank->n_experts;
        set_down_bias(a);
        jobs.push_back(a);
    }
    rc = enqueue_jobs(c, jobs);
    if (rc) return rc;
    HIPCHECK(c, weighted_sum_launch(c->stream, d, weights, experts, (uint32_t)bank->n_experts, out, (uint32_t)tokens, (uint32_t)k, (uint32_t)hidden));
    return LARQL_OK;
}

int larql_hip_dev_moe_mxfp4(larql_hip_ctx *c, const larql_hip_mxfp4_experts *bank, const float *x, size_t tokens, size_t k,
                            const uint32_t *experts, const float *weights, float *out, void *workspace, size_t workspace_bytes) {
    if (!c || !bank) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    return moe_mxfp4_block(c, bank, x, tokens, k, const_cast<uint32_t *>(experts), const_cast<float *>(weights), out, workspace,
                           workspace_bytes, nullptr, 0);  // (without logits nothing is written to experts / weights)
}

int larql_hip_dev_moe_mxfp4_routed(larql_hip_ctx *c, const larql_hip_mxfp4_experts *bank, const float *x, size_t tokens, size_t k,
                                   const float *router_logits, int policy, uint32_t *experts, float *weights, float *out,
                                   void *workspace, size_t workspace_bytes) {
    if (!c || !bank) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (k > bank->n_experts) k = bank->n_experts;  // select(): k.min(logits.len())
    if (tokens == 0 || k == 0) return LARQL_OK;
    if (bank->n_experts > kRouterMaxExperts || k > 8) return fail(c, LARQL_UNSUPPORTED, "router_select: at most 256 experts and top-8 on this backend");
    if (!router_logits) return LARQL_E_ARG;
    return moe_mxfp4_block(c, bank, x, tokens, k, experts, weights, out, workspace, workspace_bytes, router_logits, policy);
}

// ---- MoE layer: per-expert slices + split scales + router, made resident (MoeLayerWeights, pipeline/moe.rs:469-541) ----

struct larql_hip_moe_layer {
    void *region = nullptr;             // every tensor of the layer, resident
    larql_hip_mxfp4_experts bank = {};  // device pointers into `region`
    const float *router_proj = nullptr, *scale = nullptr;
    size_t n_experts = 0, top_k = 0, hidden = 0, inter = 0;
    int renormalized = 1, per_expert_scale = 0;
    // a k-quant (Q4_K / Q6_K) bank: expert e's gate rows at kq_gate + e * kq_gu_stride, its up rows at kq_up + the same,
    // its down rows at kq_down + e * kq_dn_stride; rows `cols` (gate, up) and `inter_padded` (down) elements wide
    int kq_kind = 0;  // 0: an MXFP4 bank (`bank`); else KIND_Q4K_Q8K / KIND_Q6K_Q8K, or (kq_dense) KIND_BF16 / KIND_F16 / KIND_F32
    bool kq_dense = false;
    const uint8_t *kq_gate = nullptr, *kq_up = nullptr, *kq_down = nullptr;
    uint64_t kq_gu_stride = 0, kq_dn_stride = 0;
    size_t cols = 0, inter_padded = 0;
    const float *kq_gub = nullptr, *kq_db = nullptr, *router_bias = nullptr;
    int gate_rule = 0;
    float glu_limit = 7.0f, glu_alpha = 1.702f;
    DevBuf ws, logits, rin, x, out, experts, weights;  // grown on demand (host tier: staging as well)
};

void larql_hip_moe_layer_destroy(larql_hip_ctx *c, larql_hip_moe_layer *L) {
    if (!L) return;
    if (c) { (void)hipSetDevice(c->device); (void)hipStreamSynchronize(c->stream); }
    DevBuf *bufs[] = {&L->ws, &L->logits, &L->rin, &L->x, &L->out, &L->experts, &L->weights};
    for (DevBuf *b : bufs) if (b->p) (void)hipFree(b->p);
    if (L->region) (void)hipFree(L->region);
    delete L;
}

// A Q4_K / Q6_K bank (the caller holds the context's lock): what cpu_moe_forward's integer path reads.
static int moe_layer_create_kq(larql_hip_ctx *c, const larql_hip_moe_layer_weights *w, larql_hip_moe_layer **out) {
    const size_t E = w->num_experts, hidden = w->hidden, inter = w->intermediate_size;
    // a float bank (BF16: the legacy monolith; F16, F32) takes the same way with f32 activations and the dense matvec
    // kernels (cpu_moe_forward's f32 arm, forward.rs:246-290); `blk` bytes hold `bel` elements of a row
    const bool dense = w->expert_data_format == LARQL_FMT_BF16 || w->expert_data_format == LARQL_FMT_F16 || w->expert_data_format == LARQL_FMT_F32;
    const size_t blk = dense ? (w->expert_data_format == LARQL_FMT_F32 ? 4 : 2) : w->expert_data_format == LARQL_FMT_Q6_K ? 210 : 144;
    const size_t bel = dense ? 1 : 256;
    if (w->expert_scales != LARQL_MOE_SCALES_INLINE)
        return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: a k-quant or float bank has no scale stream of its own (MoeExpertScales::Inline)");
    if (w->fused_row_layout != LARQL_MOE_ROWS_CONTIGUOUS_HALVES)
        return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: a k-quant or float bank is read as contiguous gate / up halves, as cpu_moe_forward reads it");
    if (w->gate_rule < LARQL_MOE_GATE_CLAMPED_GLU || w->gate_rule > LARQL_MOE_GATE_CLAMPED_SILU)
        return fail(c, LARQL_UNSUPPORTED, "moe_layer: unknown gate rule");
    if (w->gate_rule == LARQL_MOE_GATE_SITU_GLU && !(w->glu_limit > 0.0f))
        return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: SituGlu needs a positive beta");
    if (E == 0 || w->top_k == 0 || hidden == 0 || inter == 0) return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: empty layer");
    if (E > kRouterMaxExperts || std::min(w->top_k, E) > 8) return fail(c, LARQL_UNSUPPORTED, "moe_layer: at most 256 experts and top-8 on this backend");
    if (hidden > (1u << 24) || inter > (1u << 24)) return fail(c, LARQL_UNSUPPORTED, "moe_layer: dimensions beyond this backend");
    if (!w->experts_gate_up || !w->experts_gate_up_len || !w->experts_down || !w->experts_down_len || !w->router_proj) return LARQL_E_ARG;
    // the gate/up matrices' stored row width, from the slab length (stored_gate_up_cols, pipeline/moe.rs:659-690)
    size_t cols = hidden;
    {
        const size_t len = w->experts_gate_up_len[0];
        if (len % (2 * inter) == 0 && (len / (2 * inter)) % blk == 0 && len / (2 * inter) / blk * bel >= hidden) cols = len / (2 * inter) / blk * bel;
    }
    // MoeWeightLayout::quant_block_padded_down (moe.rs:184-200): a block format pads `inter` to whole blocks, a float format does not
    const size_t ip = dense ? inter : (inter + 255) / 256 * 256;
    if (dense) {
        if (cols % 16 != 0 || inter % 16 != 0 || cols > 8192 || inter > 8192)
            return fail(c, LARQL_UNSUPPORTED, "moe_layer: float expert rows must be multiples of 16 elements, at most 8192");
    } else {
        if (cols % 256 != 0) return fail(c, LARQL_UNSUPPORTED, "moe_layer: k-quant rows must be whole 256-element super-blocks");
        if (cols / 256 > 40 || ip / 256 > 40) return fail(c, LARQL_UNSUPPORTED, "moe_layer: k-quant rows longer than 10240 elements have no kernel");
    }
    const size_t half = inter * (cols / bel) * blk, dn = hidden * (ip / bel) * blk;
    for (size_t e = 0; e < E; e++) {
        if (!w->experts_gate_up[e] || !w->experts_down[e]) return LARQL_E_ARG;
        if (w->experts_gate_up_len[e] < 2 * half || w->experts_down_len[e] < dn)
            return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: expert %zu's slices are shorter than its geometry", e);
    }
    HIPCHECK(c, hipSetDevice(c->device));
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    // region: [gate halves | up halves | down | router_proj | router_bias | gate_up_bias | down_bias | per-expert scale]; every
    // expert's matrix starts on a 256-byte boundary (a Q6_K half is a whole number of 210-byte blocks, not of 16 bytes)
    const size_t hs = up(half), ds = up(dn);
    size_t off = 0;
    const size_t o_g = off; off += E * hs;
    const size_t o_u = off; off += E * hs;
    const size_t o_d = off; off += E * ds;
    const size_t o_rp = off; off += up(E * hidden * 4);
    const size_t o_rb = off; off += up(E * 4);
    const size_t o_gub = off; off += up(E * 2 * inter * 4);
    const size_t o_db = off; off += up(E * hidden * 4);
    const size_t o_sc = off; off += up(E * 4);
    larql_hip_moe_layer *L = new larql_hip_moe_layer();
    if (hipMalloc(&L->region, off + 64) != hipSuccess) { delete L; return fail(c, LARQL_E_DEVICE, "moe_layer: out of device memory"); }
    uint8_t *d = (uint8_t *)L->region;
    hipError_t e = hipSuccess;
    auto put = [&](size_t dst, const void *src, size_t n) {
        if (e == hipSuccess && n) e = hipMemcpyAsync(d + dst, src, n, hipMemcpyHostToDevice, c->stream);
    };
    for (size_t x = 0; x < E; x++) {
        put(o_g + x * hs, w->experts_gate_up[x], half);
        put(o_u + x * hs, w->experts_gate_up[x] + half, half);
        put(o_d + x * ds, w->experts_down[x], dn);
    }
    put(o_rp, w->router_proj, E * hidden * 4);
    if (w->router_bias) put(o_rb, w->router_bias, E * 4);
    if (w->experts_gate_up_bias) put(o_gub, w->experts_gate_up_bias, E * 2 * inter * 4);
    if (w->experts_down_bias) put(o_db, w->experts_down_bias, E * hidden * 4);
    if (w->router_per_expert_scale) put(o_sc, w->router_per_expert_scale, E * 4);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    if (e != hipSuccess) {
        (void)hipFree(L->region);
        delete L;
        return fail(c, LARQL_E_DEVICE, "moe_layer: upload: %s", hipGetErrorString(e));
    }
    L->kq_kind = dense ? kind_of_format(w->expert_data_format) : w->expert_data_format == LARQL_FMT_Q6_K ? KIND_Q6K_Q8K : KIND_Q4K_Q8K;
    L->kq_dense = dense;
    L->kq_gate = d + o_g; L->kq_up = d + o_u; L->kq_down = d + o_d;
    L->kq_gu_stride = hs; L->kq_dn_stride = ds;
    L->cols = cols; L->inter_padded = ip;
    L->kq_gub = w->experts_gate_up_bias ? (const float *)(d + o_gub) : nullptr;
    L->kq_db = w->experts_down_bias ? (const float *)(d + o_db) : nullptr;
    L->router_bias = w->router_bias ? (const float *)(d + o_rb) : nullptr;
    L->gate_rule = w->gate_rule; L->glu_limit = w->glu_limit; L->glu_alpha = w->glu_alpha;
    L->router_proj = (const float *)(d + o_rp);
    L->scale = w->router_per_expert_scale ? (const float *)(d + o_sc) : nullptr;
    L->n_experts = E; L->top_k = w->top_k; L->hidden = hidden; L->inter = inter;
    L->renormalized = w->renormalized_softmax ? 1 : 0;
    L->per_expert_scale = (w->per_expert_scale && w->router_per_expert_scale) ? 1 : 0;
    *out = L;
    return LARQL_OK;
}

int larql_hip_moe_layer_create(larql_hip_ctx *c, const larql_hip_moe_layer_weights *w, larql_hip_moe_layer **out) {
    if (!c || !w || !out) return LARQL_E_ARG;
    *out = nullptr;
    std::lock_guard<std::mutex> lk(c->mu);
    if (w->expert_data_format == LARQL_FMT_Q4_K || w->expert_data_format == LARQL_FMT_Q6_K || w->expert_data_format == LARQL_FMT_BF16 ||
        w->expert_data_format == LARQL_FMT_F16 || w->expert_data_format == LARQL_FMT_F32)
        return moe_layer_create_kq(c, w, out);
    if (w->expert_data_format != LARQL_FMT_MXFP4)
        return fail(c, LARQL_UNSUPPORTED, "moe_layer: MXFP4, Q4_K, Q6_K and float expert banks are served by this backend");
    if (w->gate_rule != LARQL_MOE_GATE_CLAMPED_GLU)
        return fail(c, LARQL_UNSUPPORTED, "moe_layer: an MXFP4 bank is served under MoeGateRule::ClampedGlu only");
    if (w->expert_scales != LARQL_MOE_SCALES_PAIRED)
        return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: an MXFP4 bank keeps its e8m0 exponents in a partner stream (MoeExpertScales::Paired)");
    const size_t E = w->num_experts, hidden = w->hidden, inter = w->intermediate_size;
    if (E == 0 || w->top_k == 0 || hidden == 0 || inter == 0) return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: empty layer");
    if (E > kRouterMaxExperts || std::min(w->top_k, E) > 8) return fail(c, LARQL_UNSUPPORTED, "moe_layer: at most 256 experts and top-8 on this backend");
    if (hidden % 32 != 0 || inter % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: hidden and intermediate_size must be multiples of 32");
    if (w->fused_row_layout != LARQL_MOE_ROWS_INTERLEAVED && w->fused_row_layout != LARQL_MOE_ROWS_CONTIGUOUS_HALVES)
        return fail(c, LARQL_E_ARG, "moe_layer: unknown fused row layout");
    if (!w->experts_gate_up || !w->experts_gate_up_len || !w->experts_down || !w->experts_down_len || !w->scales_gate_up ||
        !w->scales_gate_up_len || !w->scales_down || !w->scales_down_len || !w->router_proj)
        return LARQL_E_ARG;
    const size_t gu_p = 2 * inter * (hidden / 32) * 16, gu_s = 2 * inter * (hidden / 32);  // per expert
    const size_t dn_p = hidden * (inter / 32) * 16, dn_s = hidden * (inter / 32);
    for (size_t e = 0; e < E; e++) {
        if (!w->experts_gate_up[e] || !w->experts_down[e] || !w->scales_gate_up[e] || !w->scales_down[e]) return LARQL_E_ARG;
        if (w->experts_gate_up_len[e] < gu_p || w->scales_gate_up_len[e] < gu_s || w->experts_down_len[e] < dn_p || w->scales_down_len[e] < dn_s)
            return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: expert %zu's slices are shorter than its geometry", e);
    }
    HIPCHECK(c, hipSetDevice(c->device));
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    // region: [gate(+up) nibbles | gate(+up) exponents | down nibbles | down exponents | router_proj | router_bias |
    //          gate_up_bias | down_bias | per-expert scale], every part 256-byte aligned, 64 bytes of slack at the end
    size_t off = 0;
    const size_t o_gup = off; off += up(E * gu_p);
    const size_t o_gus = off; off += up(E * gu_s);
    const size_t o_dnp = off; off += up(E * dn_p);
    const size_t o_dns = off; off += up(E * dn_s);
    const size_t o_rp = off; off += up(E * hidden * 4);
    const size_t o_rb = off; off += up(E * 4);
    const size_t o_gub = off; off += up(E * 2 * inter * 4);
    const size_t o_db = off; off += up(E * hidden * 4);
    const size_t o_sc = off; off += up(E * 4);
    larql_hip_moe_layer *L = new larql_hip_moe_layer();
    if (hipMalloc(&L->region, off + 64) != hipSuccess) { delete L; return fail(c, LARQL_E_DEVICE, "moe_layer: out of device memory"); }
    uint8_t *d = (uint8_t *)L->region;
    const bool inter_rows = w->fused_row_layout == LARQL_MOE_ROWS_INTERLEAVED;
    hipError_t e = hipSuccess;
    auto put = [&](size_t dst, const void *src, size_t n) {
        if (e == hipSuccess && n) e = hipMemcpyAsync(d + dst, src, n, hipMemcpyHostToDevice, c->stream);
    };
    for (size_t x = 0; x < E; x++) {
        if (inter_rows) {  // the fused rows stay as stored: gate on the even, up on the odd rows, walked in place
            put(o_gup + x * gu_p, w->experts_gate_up[x], gu_p);
            put(o_gus + x * gu_s, w->scales_gate_up[x], gu_s);
        } else {
            // [gate rows | up rows] per expert: interleaved on the way up (gate row r to row 2r, up row r to row 2r+1: a
            // strided copy per half), so that the resident bank is walked as one fused matrix like a bank stored that way —
            // a one-token block then hands the gated activation from stage to stage as operand terms (20 instead of 24 us)
            const size_t rb = (hidden / 32) * 16, rs = hidden / 32;  // bytes of a row: nibbles, exponents
            auto put2d = [&](size_t dst, const uint8_t *src, size_t row) {
                if (e == hipSuccess) e = hipMemcpy2DAsync(d + dst, 2 * row, src, row, row, inter, hipMemcpyHostToDevice, c->stream);
            };
            put2d(o_gup + x * gu_p, w->experts_gate_up[x], rb);
            put2d(o_gup + x * gu_p + rb, w->experts_gate_up[x] + gu_p / 2, rb);
            put2d(o_gus + x * gu_s, w->scales_gate_up[x], rs);
            put2d(o_gus + x * gu_s + rs, w->scales_gate_up[x] + gu_s / 2, rs);
        }
        put(o_dnp + x * dn_p, w->experts_down[x], dn_p);
        put(o_dns + x * dn_s, w->scales_down[x], dn_s);
    }
    put(o_rp, w->router_proj, E * hidden * 4);
    if (w->router_bias) put(o_rb, w->router_bias, E * 4);
    if (w->experts_gate_up_bias) put(o_gub, w->experts_gate_up_bias, E * 2 * inter * 4);
    if (w->experts_down_bias) put(o_db, w->experts_down_bias, E * hidden * 4);
    if (w->router_per_expert_scale) put(o_sc, w->router_per_expert_scale, E * 4);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    if (e != hipSuccess) {
        (void)hipFree(L->region);
        delete L;
        return fail(c, LARQL_E_DEVICE, "moe_layer: upload: %s", hipGetErrorString(e));
    }
    L->bank.gate_packed = d + o_gup; L->bank.gate_scales = d + o_gus;
    L->bank.up_packed = nullptr;  // (the resident bank is interleaved whichever way the slices came)
    L->bank.up_scales = nullptr;
    L->bank.down_packed = d + o_dnp; L->bank.down_scales = d + o_dns;
    L->bank.n_experts = E; L->bank.hidden = hidden; L->bank.inter = inter;
    L->bank.limit = w->glu_limit; L->bank.alpha = w->glu_alpha;
    L->bank.gate_up_interleaved = 1;
    L->bank.router_bias = w->router_bias ? (const float *)(d + o_rb) : nullptr;
    L->bank.gate_up_bias = w->experts_gate_up_bias ? (const float *)(d + o_gub) : nullptr;
    L->bank.down_bias = w->experts_down_bias ? (const float *)(d + o_db) : nullptr;
    L->router_proj = (const float *)(d + o_rp);
    L->scale = w->router_per_expert_scale ? (const float *)(d + o_sc) : nullptr;
    L->n_experts = E; L->top_k = w->top_k; L->hidden = hidden; L->inter = inter;
    L->renormalized = w->renormalized_softmax ? 1 : 0;
    L->per_expert_scale = (w->per_expert_scale && w->router_per_expert_scale) ? 1 : 0;
    *out = L;
    return LARQL_OK;
}

// router logits on the device (one [num_experts, hidden] f32 gemv job per token), then the route and the expert block
static int moe_layer_enqueue(larql_hip_ctx *c, larql_hip_moe_layer *L, const float *router_in, const float *x, size_t tokens, float *out,
                             uint32_t *experts, float *weights) {
    const size_t E = L->n_experts, hidden = L->hidden, k = std::min(L->top_k, E);
    if (hidden % 4 != 0 || ((uintptr_t)router_in & 15) || ((uintptr_t)x & 15) || ((uintptr_t)out & 15))
        return fail(c, LARQL_REFUSED_SHAPE, "moe_layer: activations must be 16-byte aligned rows (hidden a multiple of 4)");
    const size_t wsb = L->kq_kind ? 0 : larql_hip_moe_mxfp4_workspace_bytes(tokens, k, hidden, L->inter);
    int rc = L->kq_kind ? LARQL_OK : ensure(c, L->ws, wsb); if (rc) return rc;
    rc = ensure(c, L->logits, tokens * E * 4 + 64); if (rc) return rc;
    float *logits = (float *)L->logits.p;
    std::vector<GemvJob> jobs;
    for (size_t t = 0; t < tokens; t++) jobs.push_back(make_job(KIND_F32, L->router_proj, nullptr, router_in + t * hidden, logits + t * E, E, hidden));
    rc = enqueue_jobs(c, jobs);
    if (rc) return rc;
    // softmax over all, top-k, renormalise == Router::select's NormalisedOverSelected (the same quotient of exponentials);
    // without the renormalisation the weights are the softmax's own values (SoftmaxThenSelect)
    const int policy = L->renormalized ? 1 : 0;
    if (L->kq_kind) {
        // The integer expert path of cpu_moe_forward (cpu/ops/moe/forward.rs:160-330): the route, the expert input as one
        // Q8_K activation per token at the stored row width, gate and up of every slot in one launch (the expert picked
        // from the bank at run time), the gated activation as Q8_K per slot, the down projections in one launch, and
        // the weighted sum with the down bias inside the weight.
        const size_t slots = tokens * k, inter = L->inter, ip = L->inter_padded, cols = L->cols;
        if (tokens > 65535 || slots > 65535) return fail(c, LARQL_UNSUPPORTED, "moe_layer: too many tokens in one call for a k-quant bank");
        // (a float bank: the activations stay f32 — x itself, and one row of `inter` floats per slot)
        const bool dense = L->kq_dense;
        if (dense) {
            HIPCHECK(c, router_select_launch(c->stream, logits, L->router_bias, (uint32_t)tokens, (uint32_t)E, (uint32_t)k, policy, experts, weights));
            if (L->per_expert_scale) HIPCHECK(c, expert_scale_launch(c->stream, weights, experts, L->scale, (uint32_t)slots, (uint32_t)E));
        }
        const bool pad_x = dense && cols != hidden;  // rows stored wider than hidden: x goes in zero-padded
        const size_t xq_stride = dense ? (pad_x ? cols : hidden) * sizeof(float) : (q8k_bytes(cols) + 255) & ~(size_t)255;
        const size_t aq_stride = dense ? ((inter * sizeof(float) + 255) & ~(size_t)255) : (q8k_bytes(ip) + 255) & ~(size_t)255;
        const size_t f_bytes = ((2 * slots * inter + slots * hidden) * sizeof(float) + 255) & ~(size_t)255;
        const size_t x_area = (dense && !pad_x) ? 0 : ((tokens * xq_stride + 255) & ~(size_t)255);
        rc = ensure(c, L->ws, f_bytes + x_area + slots * aq_stride + 256); if (rc) return rc;
        float *g = (float *)L->ws.p, *u = g + slots * inter, *dd = u + slots * inter;
        uint8_t *xq = (dense && !pad_x) ? (uint8_t *)const_cast<float *>(x) : (uint8_t *)L->ws.p + f_bytes;
        uint8_t *aq = (uint8_t *)L->ws.p + f_bytes + x_area;
        if (!dense)  // the route and the Q8_K expert input of every token: one launch
            HIPCHECK(c, moe_kq_route_quant_launch(c->stream, logits, L->router_bias, (uint32_t)tokens, (uint32_t)E, (uint32_t)k, policy,
                                                  L->per_expert_scale ? L->scale : nullptr, experts, weights, x, hidden, (uint32_t)hidden, (uint32_t)cols, xq,
                                                  xq_stride));
        else if (pad_x) HIPCHECK(c, pad_rows_f32_launch(c->stream, x, hidden, (uint32_t)hidden, (uint32_t)cols, (uint32_t)tokens, (float *)xq));
        jobs.clear();
        for (size_t s = 0; s < slots; s++) {
            GemvJob a = make_job(L->kq_kind, L->kq_gate, nullptr, xq + (s / k) * xq_stride, g + s * inter, inter, cols);
            a.sel = experts + s; a.w_sel_stride = L->kq_gu_stride; a.sel_count = (uint32_t)E;
            GemvJob b = a;
            b.w = L->kq_up; b.out = u + s * inter;
            jobs.push_back(a);
            jobs.push_back(b);
        }
        rc = enqueue_jobs(c, jobs);
        if (rc) return rc;
        if (dense)
            HIPCHECK(c, moe_act_f32_launch(c->stream, g, u, (uint32_t)inter, (uint32_t)slots, experts, (uint32_t)E, L->kq_gub, L->gate_rule, L->glu_limit,
                                           L->glu_alpha, (float *)aq, aq_stride / sizeof(float)));
        else
            HIPCHECK(c, moe_kq_act_q8k_launch(c->stream, g, u, (uint32_t)inter, (uint32_t)ip, (uint32_t)slots, experts, (uint32_t)E, L->kq_gub, L->gate_rule,
                                              L->glu_limit, L->glu_alpha, aq, aq_stride));
        jobs.clear();
        for (size_t s = 0; s < slots; s++) {
            GemvJob a = make_job(L->kq_kind, L->kq_down, nullptr, aq + s * aq_stride, dd + s * hidden, hidden, ip);
            a.sel = experts + s; a.w_sel_stride = L->kq_dn_stride; a.sel_count = (uint32_t)E;
            jobs.push_back(a);
        }
        rc = enqueue_jobs(c, jobs);
        if (rc) return rc;
        HIPCHECK(c, weighted_sum_bias_launch(c->stream, dd, weights, experts, (uint32_t)E, L->kq_db, out, (uint32_t)tokens, (uint32_t)k, (uint32_t)hidden));
        return LARQL_OK;
    }
    if (!L->per_expert_scale) return moe_mxfp4_block(c, &L->bank, x, tokens, k, experts, weights, out, L->ws.p, wsb, logits, policy);
    HIPCHECK(c, router_select_launch(c->stream, logits, L->bank.router_bias, (uint32_t)tokens, (uint32_t)E, (uint32_t)k, policy, experts, weights));
    HIPCHECK(c, expert_scale_launch(c->stream, weights, experts, L->scale, (uint32_t)(tokens * k), (uint32_t)E));
    return moe_mxfp4_block(c, &L->bank, x, tokens, k, experts, weights, out, L->ws.p, wsb, nullptr, 0);
}

int larql_hip_dev_moe_layer_forward(larql_hip_ctx *c, larql_hip_moe_layer *L, const float *router_in, const float *x, size_t tokens,
                                    float *out, uint32_t *experts, float *weights) {
    if (!c || !L) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (tokens == 0) return LARQL_OK;
    if (tokens > (1u << 20)) return fail(c, LARQL_UNSUPPORTED, "moe_layer: too many tokens in one call");
    if (!router_in || !x || !out || !experts || !weights) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    return moe_layer_enqueue(c, L, router_in, x, tokens, out, experts, weights);
}

int larql_hip_moe_layer_forward(larql_hip_ctx *c, larql_hip_moe_layer *L, const float *router_in, const float *x, size_t tokens,
                                float *out, uint32_t *experts_out, float *weights_out) {
    if (!c || !L) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (tokens == 0) return LARQL_OK;
    if (tokens > (1u << 20)) return fail(c, LARQL_UNSUPPORTED, "moe_layer: too many tokens in one call");
    if (!router_in || !x || !out) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    const size_t hidden = L->hidden, k = std::min(L->top_k, L->n_experts), nb = tokens * hidden * 4;
    int rc = upload(c, L->x, x, nb); if (rc) return rc;
    const float *d_rin = (const float *)L->x.p;
    if (router_in != x) { rc = upload(c, L->rin, router_in, nb); if (rc) return rc; d_rin = (const float *)L->rin.p; }
    rc = ensure(c, L->out, nb + 64); if (rc) return rc;
    rc = ensure(c, L->experts, tokens * k * 4 + 64); if (rc) return rc;
    rc = ensure(c, L->weights, tokens * k * 4 + 64); if (rc) return rc;
    Submission sub(c);
    rc = moe_layer_enqueue(c, L, d_rin, (const float *)L->x.p, tokens, (float *)L->out.p, (uint32_t *)L->experts.p, (float *)L->weights.p);
    if (rc) { (void)hipStreamSynchronize(c->stream); return rc; }
    HIPCHECK(c, hipMemcpyAsync(out, L->out.p, nb, hipMemcpyDeviceToHost, c->stream));
    if (experts_out) HIPCHECK(c, hipMemcpyAsync(experts_out, L->experts.p, tokens * k * 4, hipMemcpyDeviceToHost, c->stream));
    if (weights_out) HIPCHECK(c, hipMemcpyAsync(weights_out, L->weights.p, tokens * k * 4, hipMemcpyDeviceToHost, c->stream));
    return sub.finish();
}

// Gate-KNN over several layers in one submission (the LQL WALK / DESCRIBE shape: every layer of
// the index scored for one query, PatchedVindex::walk): one matvec launch for all layers' scores
// and one top-K launch for all (layer, position) rows.
int larql_hip_dev_gate_walk(larql_hip_ctx *c, int format, const void *const *gates, size_t n_layers, const float *x,
                            size_t x_layer_stride, size_t batch, size_t n, size_t hidden, size_t top_k, float *scores_scratch,
                            uint32_t *idx_out, float *score_out, uint32_t *count_out) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    const int kind = kind_of_format(format);
    int rc = gate_shape_check(c, kind, (size_t)-1, 0, hidden);
    if (rc) return rc;
    if (kind == KIND_Q4_0) return fail(c, LARQL_UNSUPPORTED, "gate_walk: Q4_0 gates go through larql_hip_dev_gate_knn");
    if (n_layers == 0 || batch == 0 || n == 0 || top_k == 0) return LARQL_OK;
    if (top_k > kTopkMaxK || n > 0xFFFFFFFFull || hidden == 0 || n_layers * batch > 0x7FFFFFFFull)
        return fail(c, LARQL_UNSUPPORTED, "gate_walk: unsupported size");
    if (!gates || !x || !scores_scratch || !idx_out || !score_out) return LARQL_E_ARG;
    HIPCHECK(c, hipSetDevice(c->device));
    if (!count_out) { rc = ensure(c, c->misc, n_layers * batch * 4 + 64); if (rc) return rc; count_out = (uint32_t *)c->misc.p; }
    std::vector<GemvJob> jobs;
    jobs.reserve(n_layers * batch);
    for (size_t l = 0; l < n_layers; l++)
        push_gate_jobs(jobs, kind, gates[l], x + l * x_layer_stride, batch, n, hidden, scores_scratch + l * batch * n);
    rc = enqueue_jobs(c, jobs);
    if (rc) return rc;
    HIPCHECK(c, topk_launch(c->stream, scores_scratch, (uint32_t)(n_layers * batch), (uint32_t)n, (uint32_t)top_k, true, idx_out,
                            score_out, count_out, c->nan_flag, nullptr, 0));
    return LARQL_OK;
}

// ---- device tier: encoders ---------------------------------------------------------------------

int larql_hip_dev_quantize_q4_k(larql_hip_ctx *c, const float *src, size_t n, uint8_t *dst) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_q4_k: length must be a multiple of 256");
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_q4_k_launch(c->stream, src, n, dst));
    return LARQL_OK;
}
int larql_hip_dev_quantize_q6_k(larql_hip_ctx *c, const float *src, size_t n, uint8_t *dst) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 256 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_q6_k: length must be a multiple of 256");
    if (n && ((uintptr_t)src & 15)) return fail(c, LARQL_REFUSED_SHAPE, "quantize_q6_k: the source must be 16-byte aligned");
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_q6_k_launch(c->stream, src, n, dst));
    return LARQL_OK;
}
int larql_hip_dev_quantize_q8_0(larql_hip_ctx *c, const float *src, size_t n, uint8_t *dst) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_q8_0: length must be a multiple of 32");
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_q8_0_launch(c->stream, src, n, dst));
    return LARQL_OK;
}
int larql_hip_dev_quantize_mxfp4(larql_hip_ctx *c, const float *src, size_t rows, size_t k, uint8_t *packed, uint8_t *scales) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (k % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_mxfp4: k must be a multiple of 32");
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_mxfp4_launch(c->stream, src, rows, k, packed, scales, c->log2_up));
    return LARQL_OK;
}
int larql_hip_dev_f32_to_bf16(larql_hip_ctx *c, const float *src, size_t n, uint16_t *dst) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, f32_to_bf16_launch(c->stream, src, n, dst));
    return LARQL_OK;
}
int larql_hip_dev_quantize_q4_0(larql_hip_ctx *c, const float *src, size_t n, uint8_t *dst) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    if (n % 32 != 0) return fail(c, LARQL_REFUSED_SHAPE, "quantize_q4_0: length must be a multiple of 32");
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_q4_0_launch(c->stream, src, n, dst));
    return LARQL_OK;
}
int larql_hip_dev_quantize_to_q8(larql_hip_ctx *c, const float *src, size_t n, int8_t *q8, float *scales) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, quantize_to_q8_launch(c->stream, src, n, q8, scales));
    return LARQL_OK;
}
int larql_hip_dev_fill_normal(larql_hip_ctx *c, float *dst, size_t n, uint64_t seed, float sigma) {
    if (!c) return LARQL_E_ARG;
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHECK(c, hipSetDevice(c->device));
    HIPCHECK(c, fill_normal_launch(c->stream, dst, n, seed, sigma));
    return LARQL_OK;
}

}  // extern "C"
