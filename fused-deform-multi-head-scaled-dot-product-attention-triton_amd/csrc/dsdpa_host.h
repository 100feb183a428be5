// Host-side state shared by the translation units of libdsdpa.so: error slot, kernel-path selector,
// kernel timer. Defined in dsdpa_api.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "../../include/dsdpa.h"

namespace dsdpa {

extern thread_local int g_last_hip_error;
extern std::atomic<int> g_path;

// Optional kernel timer: while enabled, every main forward/backward kernel launch carries a pair of HIP
// events. Process-wide (a framework may run the backward pass on another thread than the forward).
// The events ride on the kernel's own dispatch (hipExtLaunchKernelGGL's start/stop events: the start and
// end timestamps of that dispatch), not on hipEventRecord: an event recorded between two kernels costs
// about 5 us of idle GPU each (measured: 10 us gaps between timed kernels, none between untimed ones),
// which would make the timed step slower than the untimed one.
struct EventPair { hipEvent_t start, stop; };
struct KernelTimer {
    std::atomic<bool> on{false};
    std::mutex mu;
    std::vector<EventPair> pairs[5];   // [0] forward, [1] backward dk/dv, [2] backward dq, [3] cell binning (one pair per launch), [4] descriptor table
};
extern KernelTimer g_timer;

// One timed item: a single launch (pass start() and stop() to it) or a run of launches (start() to the
// first, stop() to the last). record = true: the item contains launches made by a library routine, which
// cannot carry events; then the pair is recorded around the run with hipEventRecord.
struct ScopedKernelTimer {
    hipStream_t st;
    EventPair ev{nullptr, nullptr};
    int which;
    bool armed = false, record;
    mutable bool handed_out = false;       // a launch took the events (or they were recorded around a run)
    ScopedKernelTimer(int which_, hipStream_t st_, bool record_ = false) : st(st_), which(which_), record(record_)
    {
        if (!g_timer.on.load(std::memory_order_relaxed)) return;
        if (hipEventCreate(&ev.start) != hipSuccess) return;
        if (hipEventCreate(&ev.stop) != hipSuccess) { (void)hipEventDestroy(ev.start); return; }
        armed = record ? hipEventRecord(ev.start, st) == hipSuccess : true;
        handed_out = record && armed;
    }
    hipEvent_t start() const { handed_out = armed; return armed && !record ? ev.start : nullptr; }
    hipEvent_t stop() const { handed_out = armed; return armed && !record ? ev.stop : nullptr; }
    ~ScopedKernelTimer()
    {
        if (!armed) return;
        if (!handed_out) {                  // the launch never happened (an early error return)
            (void)hipEventDestroy(ev.start);
            (void)hipEventDestroy(ev.stop);
            return;
        }
        if (record) (void)hipEventRecord(ev.stop, st);
        std::lock_guard<std::mutex> lock(g_timer.mu);
        g_timer.pairs[which].push_back(ev);
    }
};

// Side lane of the backward: a second stream, per host thread and device, on which the cell binning runs
// next to the dq kernel (neither needs the other; dk/dv needs both). Fork and join are events on the
// caller's stream, so the caller sees one stream's worth of ordering. Created on first use, default
// priority, never destroyed (a handful of handles per thread that ever ran a backward).
struct SideLane {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool failed = false;
};
inline SideLane *side_lane()
{
    constexpr int kMaxDevices = 64;
    thread_local SideLane lanes[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    SideLane &s = lanes[dev];
    if (s.failed) return nullptr;
    if (!s.stream) {
        if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess ||
            hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            s.failed = true;
            s.stream = nullptr;
            return nullptr;
        }
    }
    return &s;
}

// Compute units of the current device (asked once per device; 256 when the runtime will not say).
inline int device_cus()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cus[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 256;
    }
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        n = 256;
    }
    cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

inline int check_launch()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return DSDPA_ERR_HIP;
    }
    return DSDPA_OK;
}

// The plane kernels (forward, dq) keep one K and one V plane of a (b, s2, h) in LDS next to their
// per-wave descriptors; they serve every shape for which that fits in the 160 KB of a gfx950 workgroup.
constexpr size_t kLdsBytes = 160 * 1024;
constexpr size_t kPlaneDescLdsBytes = 16 * 96 * (16 + 8);   // 16 waves x 96 places x (4 weights + 2 offsets)
constexpr size_t kPlaneGradLdsBytes = 16 * 96 * 8;         // + fx, fy per place (coordinate gradient)
inline bool plane_path_fits(size_t L, size_t D, size_t esize, bool coords_grad = false)
{
    return (L + 2) * 2 * D * esize + kPlaneDescLdsBytes + (coords_grad ? kPlaneGradLdsBytes : 0) <= kLdsBytes;
}

// With very few samples per view the staged kernels mostly stage: every workgroup loads all V plane pairs for
// P samples per row and view, while the gather kernels touch only the rows they sample. Measured on 18x18,
// D = 32 (forward, staged / gather ms): V = 12: P = 2 0.344 / 0.245, P = 4 0.431 / 0.414, P = 5 0.485 / 0.516;
// V = 8: P = 3 0.173 / 0.162, P = 4 0.195 / 0.200; V = 6: equal up to P = 2, staged ahead from there.
inline bool few_samples_prefer_gather(size_t V, size_t P) { return P <= 3 && V >= 8; }

// Descriptor table of the plane kernels: per coordinate pair 16 bytes of weights and 4 of packed slot
// codes (plus, for the coordinate gradient, 16 bytes of derivative weights), computed once per call by
// plane_descriptor_kernel. Empty when the plane kernels do not apply.
struct DescLayout { size_t w, e, g, bytes; };
inline size_t round256(size_t b) { return (b + 255) / 256 * 256; }
inline DescLayout desc_layout(size_t B, size_t V, size_t Himg, size_t Wimg, size_t D, size_t P, size_t esize,
                              bool coords_grad = false)
{
    DescLayout d{0, 0, 0, 0};
    const size_t L = Himg * Wimg;
    if (!plane_path_fits(L, D, esize, coords_grad)) return d;
    const size_t m = B * V * L * V * P;
    d.w = 0;
    d.e = round256(m * 16);
    d.g = d.e + round256(m * 4);
    d.bytes = d.g + (coords_grad ? round256(m * 16) : 0);
    return d;
}

// Dense-box forward (fwd_dense_kernel): for 16-bit storage and D = 64 or 128 on shapes whose planes do not fit in LDS, with
// at least a chunk's worth of samples per view. Its workspace is one flag per tile of 16 queries, telling which
// tiles are left to the gather kernel. bytes = 0: the shape does not take that path.
struct DenseLayout { size_t todo, bytes; int ntl; };
inline DenseLayout dense_layout(size_t B, size_t V, size_t H, size_t Himg, size_t Wimg, size_t D, size_t P, size_t esize)
{
    DenseLayout d{0, 0, 0};
    const size_t L = Himg * Wimg, chunks = V * ((P + 63) / 64);
    if (esize != 2 || (D != 64 && D != 128) || P < 64 || chunks > 4096 || Himg >= 65536 || Wimg >= 65536 || plane_path_fits(L, D, esize))
        return d;
    d.ntl = (int)((L + 15) / 16);
    d.todo = 0;
    d.bytes = round256(B * H * V * (size_t)d.ntl);
    return d;
}

// Slab kernels (fwd_slab_kernel, bwd_dq_slab_kernel): fp32 storage, 16 or 32 samples per view, planes that do not fit in LDS whole but do,
// twice, as slabs of 16 columns (64 bytes per pixel, image rows at a pitch of 2 mod 4 pixels), at most 1024 pixels,
// query rows of a (batch, head) within 31 bits of coordinate pairs. Needs no workspace.
inline size_t slab_buffer_bytes(size_t Himg, size_t Wimg)
{
    const size_t pitch = Wimg + ((6 - (Wimg & 3)) & 3);
    return round256(Himg * pitch * 64);
}
inline bool slab_path_fits(size_t V, size_t Himg, size_t Wimg, size_t D, size_t P, size_t esize)
{
    const size_t L = Himg * Wimg;
    // (a wave stages runs of 16 pixels of an image row, four per slab)
    // (64 samples per view go to the gather kernels, whose window mode pays where the samples cluster)
    return esize == 4 && (P == 16 || P == 32) && (D == 32 || D == 64 || D == 128) && Himg * ((Wimg + 15) / 16) <= 64 &&
           2 * slab_buffer_bytes(Himg, Wimg) + 12 * 1024 <= kLdsBytes && !plane_path_fits(L, D, esize) &&
           V * L * V * P < ((size_t)1 << 31);
}

// Forward workspace: the descriptor table, or the dense-box forward's flags (never both).
// Backward workspace, every segment rounded up to 256 bytes:
//   delta    rows floats                     dout.out per query row
//   counters B*V*NC u32                      per (batch, key view) cell counts, then fill cursors
//   start    B*V*(NC+1) u32                  exclusive scan of the counts
//   sorted   B*V*(V*L*P) u32                 the cell lists: 12-byte records (sample id, its position (fx, fy) in the
//   frac     B*V*(V*L*P) x 8 bytes           cell) that run from `sorted` on through `frac`, which follows it; the
//                                            deterministic backward keeps plain ids in `sorted` (and sorts them)
//   items    B*V*wmax x 16 bytes             work list of the dk/dv kernel: (cell, first entry, end) per item
//   handed   bhg*V*L*(V*P) x 8 bytes         (p, sm_scale*ds) per query*sample of one GROUP of bhg (batch, head) pairs,
//                                            dq kernel -> dk/dv kernel (shapes on the gather kernels only); at most
//                                            kHandedCapBytes whatever the shape
//   acc      2*n floats                      fp32 dk/dv accumulators (16-bit storage only)
//   desc     20 bytes per coordinate pair    descriptor table (only when the plane kernels apply); 36 with
//                                            the coordinate gradient
// deterministic backward only (DSDPA_FLAG_DETERMINISTIC):
//   sorted2  as sorted                       the lists with every cell's ids in ascending order
//   seg      2*B*V*NC u32                    begin / end of every list in the flat id array
//   sorttmp  sort_temp_bytes()               scratch of the segmented sort
// with NC = (Himg+1)*(Wimg+1) cells.
size_t sort_temp_bytes(size_t n, size_t segments);                       // dsdpa_sort.hip
int sort_cell_lists(void *temp, size_t temp_bytes, const unsigned *ids_in, unsigned *ids_out, size_t n,
                    size_t segments, const unsigned *seg_begin, const unsigned *seg_end, unsigned id_bits,
                    hipStream_t st);

struct WorkspaceLayout {
    size_t delta, counters, start, sorted, frac, items, handed, handed_bytes, acc, desc, sorted2, seg, sorttmp, sorttmp_bytes, total;
    int bh_group;               // (batch, head) pairs whose pairs the handed buffer holds at a time; 0: nothing is handed over
    DescLayout dl;
    size_t counters_bytes;
    int NC;                     // cells of the grid
    int NK, vpg;                // lists per (batch, key view) = groups of query views * NC; query views per group
    unsigned piece, wmax;       // work list of the dk/dv kernel: entries per item, items per (batch, key view)
};

// Work list of the dk/dv kernel: a cell list is cut into items of at most `piece` entries, four times the
// average list length over the whole cell grid (at least 768, a multiple of 64): lists near the average
// stay whole, the heavy ones of clustered coordinates are shared by several waves. Every item ends with a flush
// of 8*D float atomics, a quarter of the kernel's time where the lists are long (64x64, 64 samples per view,
// clustered, two groups of query views: pieces of 512 entries 1.63 ms, 768 1.58, 1024 1.60, 2048 1.68 -- the last
// pieces then run alone). NC + M/piece bounds the number of items per (batch, key view), M = V*L*P being all its
// entries.
inline void work_list_geometry(size_t V, size_t L, size_t P, size_t NC, unsigned *piece, unsigned *wmax)
{
    const size_t M = V * L * P;
    size_t pc = 4 * M / NC;
    if (pc < 768) pc = 768;
    pc = (pc + 63) / 64 * 64;
    if (pc > 0x40000000u) pc = 0x40000000u;
    *piece = (unsigned)pc;
    *wmax = (unsigned)(NC + M / pc + 1);
}
// Query views per group of the dk/dv lists (only where the dq kernel hands its pairs over: there the dk/dv kernel
// waits for the query rows it gathers and for little else). The rows of one (batch, head), q and dout, are
// 2*V*L*D*e bytes; where that is more than an XCD's 4 MB of L2, the entries -- which the cell order scatters over
// all of it -- miss L2. Lists per (group of query views, cell), worked through group by group, keep the rows in
// use to one group's: groups of at most 4 MB (64x64, D = 128, 16-bit, V = 4: 8 MB, two groups: 2.31 -> 2.07 ms;
// four groups 2.23 ms -- every group multiplies the items, each with its set-up and flush), as long as the lists
// stay long enough to pay for that (an average of 48 entries over the whole grid).
inline int views_per_group(size_t V, size_t L, size_t D, size_t esize, size_t P, size_t NC, bool handed)
{
    const size_t rows_bytes = 2 * V * L * D * esize, M = V * L * P, cap = (size_t)4 << 20;
    if (!handed || rows_bytes <= cap) return (int)V;
    size_t groups = (rows_bytes + cap - 1) / cap;
    if (groups > V) groups = V;
    while (groups > 1 && M / (groups * NC) < 48) --groups;
    return (int)((V + groups - 1) / groups);
}
// The dq kernel can hand (p, sm_scale * ds) of every query*sample over to the dk/dv kernel, which then neither
// recomputes them nor needs the cell's taps. The whole backward's pairs would be rows * V*P * 8 bytes (0.54 GB
// for 2 x 4 views x 8 heads x 64x64, 64 samples per view): more than the tensors, and more than the memory-side
// cache holds. So the backward runs in GROUPS of (batch, head) pairs -- dq of a group, then dk/dv of the same
// group, the cell lists being shared by all heads -- and the buffer holds one group's pairs: at most
// kHandedCapBytes, which also stay in the memory-side cache between the two kernels. Returns the (batch, head)
// pairs per group, 0 when nothing is handed over: shapes on the staged kernels (dq and dk/dv run side by side
// there), the deterministic backward (its four colour launches recompute), one pair's samples beyond the cap or
// beyond 32-bit byte offsets.
constexpr size_t kHandedCapBytes = (size_t)128 << 20;
inline int handed_group(size_t B, size_t V, size_t H, size_t L, size_t D, size_t P, size_t esize, bool deterministic)
{
    if (deterministic || plane_path_fits(L, D, esize)) return 0;
    const size_t per_bh = V * L * (V * P) * 8;
    if (per_bh >= ((size_t)1 << 32) || per_bh > kHandedCapBytes) return 0;
    size_t g = kHandedCapBytes / per_bh;
    if (g > B * H) g = B * H;
    // groups of equal size (the last one may be smaller by less than one pair per group)
    const size_t ngroups = (B * H + g - 1) / g;
    return (int)((B * H + ngroups - 1) / ngroups);
}
inline WorkspaceLayout workspace_layout(size_t B, size_t V, size_t H, size_t Himg, size_t Wimg, size_t D, size_t P,
                                        bool storage16, bool deterministic, bool coords_grad)
{
    WorkspaceLayout w;
    const size_t rows = B * V * H * Himg * Wimg;
    w.NC = (int)((Himg + 1) * (Wimg + 1));
    size_t off = 0;
    w.delta = off; off += round256(rows * 8);           // (lse, delta) per row
    w.bh_group = handed_group(B, V, H, Himg * Wimg, D, P, storage16 ? 2 : 4, deterministic);
    const bool handed = w.bh_group > 0;
    w.vpg = views_per_group(V, Himg * Wimg, D, storage16 ? 2 : 4, P, (size_t)w.NC, handed);
    w.NK = w.NC * (int)((V + w.vpg - 1) / w.vpg);
    w.counters = off; w.counters_bytes = round256(B * V * (size_t)w.NK * 4); off += w.counters_bytes;
    w.start = off; off += round256(B * V * ((size_t)w.NK + 1) * 4);
    w.sorted = off; off += round256(B * V * (V * Himg * Wimg * P) * 4);
    w.frac = off; off += round256(B * V * (V * Himg * Wimg * P) * 8);
    work_list_geometry(V, Himg * Wimg, P, (size_t)w.NK, &w.piece, &w.wmax);
    w.items = off; off += round256(B * V * (size_t)w.wmax * 16);
    // (p, sm_scale * ds) per query*sample of one group of (batch, head) pairs, handed from the dq kernel to the
    // dk/dv kernel (see handed_group)
    w.handed = off;
    w.handed_bytes = round256((size_t)w.bh_group * V * Himg * Wimg * (V * P) * 8);
    off += w.handed_bytes;
    w.acc = off; if (storage16) off += round256(2 * rows * D * 4);
    // with the coordinate gradient the staged dq kernel needs more LDS; where it no longer fits, dq takes the
    // gather kernel and no table is needed
    w.dl = desc_layout(B, V, Himg, Wimg, D, P, storage16 ? 2 : 4, coords_grad);
    w.desc = off; off += w.dl.bytes;
    w.sorted2 = w.seg = w.sorttmp = off;
    w.sorttmp_bytes = 0;
    if (deterministic) {
        const size_t ids = B * V * (V * Himg * Wimg * P), segs = B * V * (size_t)w.NC;
        w.sorted2 = off; off += round256(ids * 4);
        w.seg = off; off += round256(2 * segs * 4);
        w.sorttmp_bytes = round256(sort_temp_bytes(ids, segs));
        w.sorttmp = off; off += w.sorttmp_bytes;
    }
    w.total = off;
    return w;
}

// One storage type's forward / backward entry (argument checks, kernel selection, launches); each is
// instantiated in its own translation unit (dsdpa_f32.hip, dsdpa_bf16.hip, dsdpa_f16.hip) so that the
// three compile in parallel.
// `strides`: null (everything contiguous) or the 8 element strides of q and of k/v over (batch, view, head, pixel).
// dense_ok: the workspace has room for dense_layout() (false: the gather kernels alone do those shapes).
template <typename S>
int fwd_impl(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
             void *workspace, int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale,
             const long long *strides, void *stream, bool dense_ok = true);
template <typename S>
int bwd_impl(const void *q, const void *k, const void *v, const float *coords, const void *out,
             const float *lse, const void *dout, void *dq, void *dk, void *dv, float *dcoords, void *workspace,
             int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides,
             unsigned flags, void *stream);

}  // namespace dsdpa
