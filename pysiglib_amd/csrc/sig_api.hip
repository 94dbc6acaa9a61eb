// C ABI of the MI355X signature library: the four hot entry points of the
// reference's GPU plugin (siglib/cusig/cu_signature.cu:3494-3545) plus its
// lifecycle symbols, re-implemented on the gfx950 tree kernels.
//
// Every entry point is synchronous (device work has completed on return), never
// throws across the ABI, returns the reference's status codes
// (siglib/cusig/cu_macros.h:27-89) and leaves a message in a thread-local buffer
// (siglib/shared/last_error.h:22-41).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <charconv>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/cusig_amd.h"
#include "sig_chen_adjoint.h"
#include "sig_deep.h"
#include "sig_rows.h"
#include "sig_degree2.h"
#include "sig_degree3.h"
#include "sig_host.h"
#include "sig_kernels.h"
#include "sig_registry.h"

namespace sigamd {

thread_local char g_last_error[4096] = {0};

// ---------------------------------------------------------------------------
// kernel table
// ---------------------------------------------------------------------------
struct Table {
    // several partitions (tail, k) of one shape may be compiled; the first listed is the default
    std::map<std::tuple<int, int, int>, std::vector<const KernelEntry*>> fwd, bwd;
    Table()
    {
        int n = 0;
        const EntryList* lists = all_entry_lists(&n);
        for (int i = 0; i < n; ++i)
            for (int j = 0; j < lists[i].count; ++j) {
                const KernelEntry* e = &lists[i].entries[j];
                auto key = std::make_tuple(e->is_f64, e->D, e->N);
                auto& slot = e->fwd ? fwd[key] : bwd[key];
                if (e->preferred && !e->staged) slot.insert(slot.begin(), e);
                else slot.push_back(e);
            }
    }
};

// Process-wide hooks (tuning, tests, measurement) may be set by one thread while another is inside a call: atomics,
// read once where a call needs a consistent value.
using Hook = std::atomic<int>;
// the tuning and test hooks below only take effect after cusig_amd_enable_test_hooks(1): a caller that merely links
// the library cannot reroute the kernels of other threads by accident
static Hook g_test_hooks{0};
// tuning hook: when set (tail > 0), prefer the compiled partition with this (tail, k)
static Hook g_force_tail{0}, g_force_k{0};
static Hook g_ignore_table{0};          // tuning hook: every shape runs the run-time-dimension kernels, as if it had no compiled instance
static Hook g_force_run_time_wide{0};   // with a forced partition: take the run-time-dimension kernel in the wide layout

static const Table& table()
{
    static const Table t;
    return t;
}

static int simd_count();
static const KernelEntry* find_entry(bool backward, bool f64, uint64_t d, uint64_t degree);
static double sweep_estimate(const KernelEntry* e, int d, int64_t batch, int64_t L, bool backward);

// The specialised partition of a shape is tuned for a full chip; with few paths its few, heavy lanes make every
// one of the L dependent steps slow.  Then the run-time-dimension kernel (one word prefix per lane, many light
// lanes) finishes sooner even though it issues more instructions in total.
static const KernelEntry* choose_entry(bool backward, bool f64, uint64_t d, uint64_t degree, uint64_t batch, uint64_t L)
{
    const KernelEntry* spec = find_entry(backward, f64, d, degree);
    if (!spec || spec->D == 0 || g_force_tail > 0) return spec;
    const auto& m = backward ? table().bwd : table().fwd;
    auto it = m.find(std::make_tuple(int(f64), 0, int(degree)));
    if (it == m.end() || it->second.empty()) return spec;
    const KernelEntry* gen = it->second.front();
    return sweep_estimate(gen, int(d), int64_t(batch), int64_t(L), backward) <
                   0.7 * sweep_estimate(spec, int(d), int64_t(batch), int64_t(L), backward)
               ? gen
               : spec;
}

// Shapes without a specialised instance run a run-time-dimension kernel.  Its default carries few depth-1 letters
// per lane in the packed layout, which suits the few lanes of small shapes.  Up to degree 10 there are variants with
// more letters per lane (the chain work of a lane is shared by more top-level updates), most of them in the wide
// layout (one letter group of one path per wave, the group's increments arriving through scalar loads), which needs
// at least 48 word prefixes.  Measured for d = 41 .. 80 at degree 4, 21 .. 32 at degree 5, 9 .. 16 at degree 6,
// 6 .. 8 at degree 7 and 5 .. 6 at degree 8: 2-16x faster forward, 1.5-5x backward than the default.
static const KernelEntry* pick_run_time_entry(bool backward, bool f64, int d, int degree)
{
    const auto& m = backward ? table().bwd : table().fwd;
    auto packed = m.find(std::make_tuple(int(f64), 0, degree));
    if (packed == m.end() || packed->second.empty()) return nullptr;
    const KernelEntry* best = packed->second.front();
    const KernelEntry* packed_many = nullptr;
    for (const KernelEntry* e : packed->second)
        if (e->k > best->k && !e->staged && (!packed_many || e->k > packed_many->k)) packed_many = e;
    auto wide = m.find(std::make_tuple(int(f64), -1, degree));
    if (wide == m.end() || wide->second.empty() || ipow64(d, degree - 1) < 48)
        return d >= 12 && packed_many ? packed_many : best;
    // single precision backward at 9 .. 15 channels: the packed 16-letter variant is ~10 % ahead of the wide one,
    // whose only letter group is then partly empty
    if (backward && !f64 && d > 8 && d < 16 && packed_many) return packed_many;
    // letters per lane: a partly empty last group costs more than the longer chain share of a smaller K
    // (forward, 32 letters: single precision only -- a double-precision row of 32 does not fit the scalar registers twice)
    const int want = d <= 8 ? 8 : backward ? (d <= 32 ? 16 : 32) : (d % 32 == 0 && !f64 ? 32 : 16);
    const KernelEntry* pick = nullptr;
    for (const KernelEntry* e : wide->second) {
        if (e->staged) continue;
        // the largest letter count up to `want`, else the smallest there is
        if (!pick || (e->k <= want ? (pick->k > want || e->k > pick->k) : (pick->k > want && e->k < pick->k))) pick = e;
    }
    return pick ? pick : best;
}

static const KernelEntry* find_entry(bool backward, bool f64, uint64_t d, uint64_t degree)
{
    const auto& m = backward ? table().bwd : table().fwd;
    if (d <= 0x7fffffff && degree <= 0x7fffffff) {
        auto it = m.find(std::make_tuple(int(f64), int(d), int(degree)));
        const bool run_time = it == m.end() || g_ignore_table != 0;
        if (run_time) it = m.find(std::make_tuple(int(f64), 0, int(degree)));
        if (it != m.end() && !it->second.empty()) {
            if (g_force_tail > 0) {
                auto from = it;
                if (run_time && g_force_run_time_wide && ipow64(int64_t(d), int(degree) - 1) >= 48) {
                    auto w = m.find(std::make_tuple(int(f64), -1, int(degree)));
                    if (w != m.end()) from = w;
                }
                for (const KernelEntry* e : from->second)
                    if (e->tail == g_force_tail && e->k == g_force_k && !e->staged) return e;
            }
            if (run_time) return pick_run_time_entry(backward, f64, int(d), int(degree));
            return it->second.front();
        }
    }
    return nullptr;
}

// Rough VALU instruction count of one forward step of one lane for partition (tail, k); the backward costs a
// near-constant multiple of it, so the same figure ranks partitions for both sweeps.
static double lane_step_cost(int d, int n, int tail, int k)
{
    const int m = n - tail;
    double cost = m;
    for (int t = 1; t <= n; ++t) {
        if (t == 1) cost += 1;
        else if (t <= m) cost += 2.0 * (t - 1);
        else {
            cost += 1 + 2.0 * (m - 1);
            double nodes = k;
            for (int e = 1; e <= t - m; ++e) {
                cost += (e == t - m) ? nodes : 2.0 * nodes + nodes / (e == 1 ? k : d);
                nodes *= d;
            }
        }
    }
    return cost;
}

// A sweep is a chain of dependent steps: its duration is their number times the longer of one lane-step (latency
// of a lone wave) and the chip-wide issue time of all waves' steps.  Long paths of an under-filled launch are cut
// in time (about two waves per SIMD, segments of at least 32 resp. 48 steps), which divides the chain and multiplies
// the waves.  Returns a relative figure.
static double sweep_estimate(const KernelEntry* e, int d, int64_t batch, int64_t L, bool backward)
{
    const TreeGeom g = make_geom(d, e->N - e->tail, e->k, e->D != 0);
    const double waves = double(total_waves(g, batch));
    const double simds = double(simd_count());
    double cuts = 1.0;
    if (waves * 2 <= simds) cuts = std::max(1.0, std::min({2.0 * simds / waves, double(L / (backward ? 32 : 48)), backward ? 64.0 : 32.0}));
    const double per_step = lane_step_cost(d, e->N, e->tail, e->k) * (e->D > 0 ? 1.0 : 1.15);
    return per_step / cuts * std::max(1.0, waves * cuts / simds * 0.8);
}

// the LDS-staged twin of a kernel instance (same partition), if one was compiled
static const KernelEntry* staged_twin(bool backward, const KernelEntry* base)
{
    const auto& m = backward ? table().bwd : table().fwd;
    auto it = m.find(std::make_tuple(base->is_f64, base->D, base->N));
    if (it == m.end()) return nullptr;
    for (const KernelEntry* e : it->second)
        if (e->staged && e->tail == base->tail && e->k == base->k) return e;
    return nullptr;
}

// ---------------------------------------------------------------------------
// per-device workspace (grow-only; released by cusig_shutdown).  The mutex also
// serialises concurrent host threads on the shared buffers, as the reference
// does for its backward workspaces (siglib/cusig/cu_signature.cu:2971).
// ---------------------------------------------------------------------------
struct Workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
};
std::atomic<int> g_force_wide_index{0};
std::atomic<int> g_chen_adjoint_mode{0};
std::atomic<int> g_chen_low_levels{1};
std::mutex g_ws_mutex;
static std::map<std::pair<int, int>, Workspace> g_ws;   // (device, slot)

// test hook: workspace requests above this many bytes fail as if the device were out of memory (0: no limit)
static std::atomic<uint64_t> g_alloc_limit{0};
static std::atomic<int> g_alloc_retries{0};     // calls split in two after a failed workspace allocation

void* workspace(int slot, size_t bytes)
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    Workspace& w = g_ws[{dev, slot}];
    if (w.bytes < bytes) {
        if (w.ptr) {
            SIG_HIP(hipFree(w.ptr));
            w.ptr = nullptr;
            w.bytes = 0;
        }
        const size_t want = (bytes + bytes / 8 + 255) & ~size_t(255);
        const uint64_t limit = g_alloc_limit;
        if ((limit && want > limit) || hipMalloc(&w.ptr, want) != hipSuccess) {
            (void)hipGetLastError();
            w.ptr = nullptr;
            throw std::bad_alloc();
        }
        w.bytes = want;
    }
    return w.ptr;
}

// The increment-gradient accumulators of backward sweeps that form their own increments (no pre-pass launch that could
// clear one): two buffers per device take turns.  The launch that turns a call's accumulator into the path gradient also
// clears whatever the other buffer still holds, so the next call finds its accumulator zero.  `dirty` counts the leading
// bytes that may be non-zero (everything after an allocation; a failed call leaves its buffer dirty and `next`
// unchanged, and the next call clears it with a launch of its own).  Guarded by the workspace mutex.
struct DzPair {
    void* ptr[2] = {nullptr, nullptr};
    size_t capacity[2] = {0, 0};
    size_t dirty[2] = {0, 0};
    int next = 0;
};
static std::map<int, DzPair> g_dz;      // per device
constexpr int kDzSlot[2] = {16, 17};

static void* dz_pair_buffer(DzPair& st, int which, size_t bytes)
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    void* p = workspace(kDzSlot[which], bytes);
    const size_t capacity = g_ws[{dev, kDzSlot[which]}].bytes;
    if (p != st.ptr[which] || capacity != st.capacity[which]) {     // fresh memory: all of it may be non-zero
        st.ptr[which] = p;
        st.capacity[which] = capacity;
        st.dirty[which] = capacity;
    }
    return p;
}

static int* g_flag_host = nullptr;     // pinned word the forward kernels report NaN / infinity through

static void release_workspaces() noexcept
{
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    for (auto& kv : g_ws) {
        if (kv.second.ptr) {
            int cur = 0;
            if (hipGetDevice(&cur) == hipSuccess && hipSetDevice(kv.first.first) == hipSuccess) {
                (void)hipFree(kv.second.ptr);
                (void)hipSetDevice(cur);
            }
        }
    }
    g_ws.clear();
    g_dz.clear();
    rocblas_release();
    if (g_flag_host) {
        (void)hipHostFree(g_flag_host);
        g_flag_host = nullptr;
    }
    (void)hipGetLastError();
}

// ---------------------------------------------------------------------------
// kernel timing hook for the benchmark
// ---------------------------------------------------------------------------
static std::atomic<bool> g_profile{false};
static std::atomic<float> g_last_ms{-1.f};
// name and events are only touched under the workspace mutex (every timer lives inside a locked region)
static char g_last_name[128] = {0};
static hipEvent_t g_ev0 = nullptr, g_ev1 = nullptr;

struct MainKernelTimer {
    hipStream_t s;
    bool on;
    MainKernelTimer(hipStream_t stream, const char* name, bool allowed = true) : s(stream), on(g_profile && allowed)
    {
        if (!on) return;
        if (!g_ev0) {
            SIG_HIP(hipEventCreate(&g_ev0));
            SIG_HIP(hipEventCreate(&g_ev1));
        }
        std::snprintf(g_last_name, sizeof g_last_name, "%s", name);
        SIG_HIP(hipEventRecord(g_ev0, s));
    }
    // defer: only mark the end; read() fetches the duration later, so that kernels enqueued after the timed one do
    // not wait for a host round trip
    void stop(bool defer = false)
    {
        if (!on) return;
        SIG_HIP(hipEventRecord(g_ev1, s));
        if (!defer) read();
    }
    void read()
    {
        if (!on) return;
        SIG_HIP(hipEventSynchronize(g_ev1));
        float ms = -1.f;
        SIG_HIP(hipEventElapsedTime(&ms, g_ev0, g_ev1));
        g_last_ms = ms;
    }
};

// Stream-ordered mode (off by default): signature_cuda / sig_backprop_cuda only enqueue their kernels on the null
// stream and return; neither the device-wide wait on entry nor the wait for completion is made.  Correct for callers
// whose producers and consumers are ordered with the null stream (PyTorch's default stream is the null stream, and
// blocking streams synchronise with it implicitly); it removes the host round trip between consecutive calls.
static Hook g_stream_ordered{0};
static void entry_sync()
{
    if (!g_stream_ordered) SIG_HIP(hipDeviceSynchronize());
}
static void exit_sync(hipStream_t stream)
{
    if (!g_stream_ordered) SIG_HIP(hipStreamSynchronize(stream));
}

// ---------------------------------------------------------------------------
// NaN / infinity report of the forward pass
// ---------------------------------------------------------------------------
// The kernels that store a signature set a flag when a stored value is not finite, so that callers who must warn
// about overflow (pysiglib/sig.py:299-311 scans the result for NaN and Inf) need no pass of their own over the
// output.  The flag is one word of pinned host memory mapped into the device: it costs nothing to read after the
// call's final synchronisation.  Calls are serialised by the workspace mutex; each thread keeps its own last answer.
static thread_local int tl_sig_nonfinite = -1;     // -1: the last forward call on this thread did not report

static int* nonfinite_flag()
{
    if (!g_flag_host) SIG_HIP(hipHostMalloc(reinterpret_cast<void**>(&g_flag_host), 64, hipHostMallocMapped | hipHostMallocPortable));
    int* dev = nullptr;
    SIG_HIP(hipHostGetDevicePointer(reinterpret_cast<void**>(&dev), g_flag_host, 0));
    return dev;
}

// ---------------------------------------------------------------------------
// time segmentation of the forward sweep
// ---------------------------------------------------------------------------
static Hook g_force_segments{0};   // tuning hook (0 = automatic)
static thread_local int tl_last_segments = 0;   // pieces per path of the last forward sweep on this thread (0: no sweep ran)
static Hook g_point_fed{1};        // tuning hook: 0 always computes the increments in a kernel of their own
static Hook g_lead_lag_sparse{1};  // tuning hook: 0 sweeps lead-lag paths like any other (every letter of every step)

static int simd_count()
{
    static int cached = 0;
    if (!cached) {
        int dev = 0, cus = 0;
        SIG_HIP(hipGetDevice(&dev));
        SIG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        cached = 4 * (cus > 0 ? cus : 256);
    }
    return cached;
}

// Cutting every path into g pieces of 1/g of the steps multiplies the waves and divides the chain of dependent
// steps; it costs one signature write per piece plus the Chen folds.  Two situations pay:
//  * under-filled: whole-path sweeps leave SIMDs without a wave (few paths);
//  * unevenly filled: a few waves per SIMD, and the fullest SIMD holds one more than most (1280 waves on 1024 SIMDs
//    that hold two each run as long as 2048 would); the launch lasts as long as its fullest SIMD needs, and shorter
//    pieces even the load out.
// A small model picks g: the fullest SIMD works through its waves `waves_per_simd` at a time, a SIMD with two or
// more resident waves issuing `pair_rate` times as fast as with one; a step of a lone wave takes 2.4 ns per
// instruction of lane_step_cost, and at least 240 ns when its increments come straight from memory instead of the
// LDS ring (lane_step(g) says which, for the launch g pieces make); the folds cost a fixed 8 us, 10 us per launch
// and 2.2 signature sets of traffic per piece at 4 TB/s (measured: d = 12, degree 4, 48 paths of 300 steps: whole
// 92 us, 2 pieces 77, 3: 76, 4: 94, 6: 101 us).  Pieces keep at least 48 steps and 256 MB of segment signatures at most, and a
// split must promise 7 % (batch 128, length 1024, d = 5, degree 7, f32: 0.587 -> 0.523 ms with three pieces).
template <typename LaneStep>
static int choose_segments(int64_t waves, int64_t L, int waves_per_simd, uint64_t sig_bytes_all_paths, LaneStep&& lane_step,
                           bool f64)
{
    const int64_t simds = simd_count();
    if (waves <= 0 || sig_bytes_all_paths == 0) return 1;
    const int occ = std::max(1, waves_per_simd);
    if (waves > 4 * simds * occ) return 1;
    const double pair_rate = f64 ? 1.2 : 1.35;
    auto estimate = [&](int g) {
        const int64_t fullest = (waves * g + simds - 1) / simds;          // waves of the fullest SIMD
        const int64_t rounds = fullest / occ, rest = fullest % occ;
        double steps = double(rounds) * occ / (occ > 1 ? pair_rate : 1.0);
        if (rest) steps += double(rest) / (rest > 1 ? pair_rate : 1.0);
        double t = double((L + g - 1) / g) * lane_step(g) * steps;
        if (g > 1) {
            int launches = 0;
            for (int m = g; m > 1; m = (m + 1) / 2) ++launches;
            t += 8e-6 + 10e-6 * launches + 2.2 * g * double(sig_bytes_all_paths) / 4e12;
        }
        return t;
    };
    int best = 1;
    double best_t = estimate(1);
    const double whole = best_t;
    // (one very long path of few channels: hundreds of pieces, each further doubling one more 10 us fold)
    for (int g : {2, 3, 4, 5, 6, 8, 10, 12, 16, 20, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024}) {
        if (L / g < 48 || uint64_t(g) * sig_bytes_all_paths > (uint64_t(256) << 20)) break;
        const double t = estimate(g);
        if (t < best_t) { best = g; best_t = t; }
    }
    return best_t < 0.93 * whole ? best : 1;
}

// The backward sweep can be cut in time as well: the state at the end of segment g is the Chen product of the
// segment signatures up to g, and the adjoint of that state is the upstream gradient pulled back through the product
// with the remaining segments.  That costs a segmented forward sweep, two chains of Chen products and one product
// adjoint, all over (path, segment) rows.
static Hook g_force_bwd_segments{0};   // tuning hook (0 = automatic)
static Hook g_rows_forward{1};         // test hook: the same for the forward sweep
static Hook g_rows_backward{1};        // test hook: 0 = shapes beyond the table never take the by-row reverse sweep (sig_rows.hip)

// g pieces are chosen by the same kind of model as for the forward sweep (fullest SIMD, `pair_rate`, lane_step(g) =
// seconds per step of a lone wave).  The extra work is larger here: the segmented forward sweep (a third of the
// backward's arithmetic), 2 ceil(log2 g) + 2 launches of about 10 us each on top of a fixed 30 us, and the
// traffic of the scans and of the product adjoint over g rows per path, fitted at 4.2 + 0.64 ceil(log2 g) ps per
// byte of segment signatures (48 paths of 300 steps, d = 12, degree 4, f64: whole 0.225 ms, 2 pieces 0.270,
// 8: 0.578, 64: 4.65 ms; 8 paths of 4000 steps, d = 6, degree 4, f32: whole 3.42 ms, 32 pieces 0.249 ms).
template <typename LaneStep>
static int choose_bwd_segments(int64_t waves, int64_t L, int waves_per_simd, uint64_t sig_bytes_all_paths, LaneStep&& lane_step,
                               bool f64)
{
    const int64_t simds = simd_count();
    if (waves <= 0 || sig_bytes_all_paths == 0) return 1;
    const int occ = std::max(1, waves_per_simd);
    if (waves > 2 * simds * occ) return 1;
    const double pair_rate = f64 ? 1.2 : 1.35;
    auto estimate = [&](int g) {
        const int64_t fullest = (waves * g + simds - 1) / simds;
        const int64_t rounds = fullest / occ, rest = fullest % occ;
        double steps = double(rounds) * occ / (occ > 1 ? pair_rate : 1.0);
        if (rest) steps += double(rest) / (rest > 1 ? pair_rate : 1.0);
        double t = double((L + g - 1) / g) * lane_step(g) * steps;
        if (g > 1) {
            int lg = 0;
            while ((1 << lg) < g) ++lg;
            t *= 1.31;
            t += 30e-6 + 10e-6 * (2 * lg + 2) + double(g) * double(sig_bytes_all_paths) * (4.2e-12 + 0.64e-12 * lg);
        }
        return t;
    };
    int best = 1;
    double best_t = estimate(1);
    const double whole = best_t;
    for (int g : {2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512}) {
        if (L / g < 32 || uint64_t(g) * sig_bytes_all_paths > (uint64_t(64) << 20)) break;
        const double t = estimate(g);
        if (t < best_t) { best = g; best_t = t; }
    }
    return best_t < 0.93 * whole ? best : 1;
}

// With at most two waves per SIMD the LDS-staged twin (all-VGPR FMAs, HBM latency hidden by a chunk of
// arithmetic) is the faster way to feed increments.  With more resident waves it depends (measured over d = 4..24,
// degrees 4..6, 3-9 waves per SIMD): the f32 forward is always faster staged (1.2-1.8x: SGPR-operand FMAs issue
// slower than all-VGPR ones), the f32 backward up to 13 channels and both f64 sweeps up to 8 (1.05-1.3x), while with
// more channels the ring's LDS reads cost them 3-30 % (f64 at 10-12 channels is mixed).
static Hook g_force_staged{-1};   // tuning hook: -1 automatic, 0 never, 1 whenever compiled

// lead_lag_sparse: the path is a lead-lag path and staged twins that skip a step's still letters may be used.  Those
// twins do about 40 % less arithmetic, which outweighs what the tuned choice for dense paths says: measured on 144
// lead-lag shapes (2-20 raw channels, both precisions), the forward twin is faster wherever it exists (mean 0.82x), the
// backward twin in single precision and, in double precision, up to 13 augmented channels (mean 0.85x; beyond, its
// register pressure costs more than the skipped work saves, and the general rules below decide; the scalar-fed
// backward kernels of those dimensions have a lead-lag form of their own).
static const KernelEntry* pick_variant(bool backward, const KernelEntry* base, int64_t waves, bool lead_lag_sparse = false)
{
    if (lead_lag_sparse && g_force_staged < 0) {
        const KernelEntry* twin = base->staged ? base : staged_twin(backward, base);
        if (twin && (backward ? (twin->bwd_lead_lag && (!twin->is_f64 || twin->D <= 13)) : twin->fwd_lead_lag != nullptr))
            return twin;
    }
    const bool small_dim = base->D > 0 && base->D <= (base->is_f64 ? 8 : 13);
    const bool want = g_force_staged >= 0 ? g_force_staged != 0
                      : base->stage_policy == 1 ? true
                      : base->stage_policy == 2 ? false
                      : base->stage_policy == 3 ? waves <= 2 * int64_t(simd_count())
                                                : waves <= 2 * int64_t(simd_count()) || small_dim ||
                                                      (!backward && !base->is_f64);
    if (!want) return base;
    const KernelEntry* twin = staged_twin(backward, base);
    return twin ? twin : base;
}

// ---------------------------------------------------------------------------
// degree 2 in closed form (matrix cores): taken for paths of many channels, where no specialised sweep exists
// ---------------------------------------------------------------------------
static Hook g_force_degree2{-1};    // tuning hook: -1 automatic, 0 never, 1 whenever the degree is 2
static Hook g_degree2_staged{1};    // tuning hook: 0 keeps the operands of the degree-2 products out of LDS

// Measured against the sweeps for d = 3 .. 256: the backward wins everywhere (1.4x at d = 4, 20x at d = 64), the
// forward from about 12 channels on and for small dimensions whenever the sweeps cannot fill the chip.
static Hook g_force_degree3{-1};    // tuning hook: -1 automatic, 0 never, 1 whenever the degree is 3
// rows buffer [paths of a chunk][L][d^2] of the degree-3 matrix form: paths are taken in chunks that fit this many bytes
constexpr uint64_t kDeg3BufBytes = uint64_t(1) << 30;

// degree 3 as library matrix products around a scan (sig_degree3.h): two products backward, one forward.  Measured at
// batch 512 (256 at 128 channels), length 256, backward, against the by-row reverse sweep (which needs neither the
// library nor the rows buffer): float32 48 channels 2.96 / 2.80 ms, 64: 4.23 / 4.27, 80: 9.3 / 19.4, 128: 9.2 / 15.6;
// float64 64 channels 6.8 / 9.8, 80: 14.6 / 35.5, 128: 27.0 / 40.8 (below 48 channels the compiled float64 instances:
// 1.3x from 36).  The scan needs a wave per SIMD to be worth it (a wave: 8 rows x 64 columns of one path's level 2).
static bool want_degree3_gemm(uint64_t d_aug, uint64_t degree, uint64_t L, uint64_t batch, bool f64, bool backward)
{
    if (degree != 3 || d_aug < 2 || d_aug > uint64_t(kDeg3MaxDim) || L > 0x7fffffff) return false;
    // one path's rows must fit the buffer (longer paths stay with the sweeps, which need B * L * d elements)
    if (L > kDeg3BufBytes / (d_aug * d_aug * (f64 ? 8 : 4))) return false;
    if (g_force_degree3 >= 0) return g_force_degree3 != 0;
    const uint64_t waves = ((d_aug + kWave - 1) / kWave) * ((d_aug + kDeg3RowsPerThread - 1) / kDeg3RowsPerThread) * batch;
    const uint64_t from = backward ? (f64 ? 36u : 65u) : 112u;      // forward: 1.3x at 128 channels, slower at 80
    return d_aug >= from && waves >= 1024;
}

static bool use_degree2(bool backward, uint64_t d_aug, uint64_t degree, uint64_t batch)
{
    if (degree != 2 || d_aug < 2 || d_aug > 0x7fff) return false;
    if (g_force_degree2 >= 0) return g_force_degree2 != 0;
    return backward || d_aug >= 12 || batch * 8 <= uint64_t(simd_count());
}

// ---------------------------------------------------------------------------
// degrees beyond the instance table: run-time-degree sweeps (sig_deep.hip)
// ---------------------------------------------------------------------------
static Hook g_force_deep{0};        // test hook: 1 takes the run-time-degree sweeps wherever they apply

static bool use_deep(uint64_t d_aug, uint64_t degree)
{
    if (!deep_supported(d_aug, degree)) return false;
    return degree > 16 || g_force_deep != 0;
}

// the reference's run-time-degree kernels stop at degree 64 (siglib/cusig/cu_signature.cu:400,3022-3025)
static void check_degree_limit(uint64_t d_aug, uint64_t degree, const char* who)
{
    if (d_aug >= 2 && degree > uint64_t(kDeepMaxDegree))
        throw std::invalid_argument(std::string(who) + " requires degree <= 64. Use CPU or reduce the truncation level.");
}

// ---------------------------------------------------------------------------
// shared argument handling
// ---------------------------------------------------------------------------
static void validate_correction(const void* correction, uint64_t correction_len, uint64_t dimension,
                                uint64_t degree, bool lead_lag)
{
    // siglib/cpsig/cp_signature.h:229-256
    if (correction == nullptr && correction_len != 0)
        throw std::invalid_argument("correction pointer is null but correction_len is nonzero");
    if (lead_lag && correction_len != 0)
        throw std::invalid_argument("correction cannot be used with lead_lag=true");
    if (correction_len == 0) return;
    if (degree < 2) throw std::invalid_argument("correction must be empty when degree < 2");
    uint64_t offset = 0, level_size = dimension;
    bool ok = false;
    for (uint64_t level = 2; level <= degree; ++level) {
        level_size *= dimension;
        offset += level_size;
        if (offset == correction_len) { ok = true; break; }
        if (offset > correction_len) break;
    }
    if (!ok) throw std::invalid_argument("correction length must be a prefix of tensor levels 2..degree");
    throw std::runtime_error("per-segment correction is not implemented in this build");
}

struct Shape {
    uint64_t d_aug, len_aug, L, full_len, stride;
};

static Shape make_shape(uint64_t dimension, uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                        bool scalar_term)
{
    Shape s;
    s.d_aug = (lead_lag ? 2 * dimension : dimension) + (time_aug ? 1 : 0);
    s.len_aug = (lead_lag && length > 0) ? 2 * length - 1 : length;
    s.L = s.len_aug > 0 ? s.len_aug - 1 : 0;
    s.full_len = sig_length_u64(s.d_aug, degree);
    if (s.full_len == 0) throw std::overflow_error("signature length overflows 64 bits");
    s.stride = scalar_term ? s.full_len : s.full_len - 1;
    return s;
}

template <typename T>
static void compute_increments(const T* path, T* inc, uint64_t batch, uint64_t dimension, uint64_t length,
                               bool time_aug, bool lead_lag, T end_time, const Shape& s, hipStream_t stream,
                               T* zero_out = nullptr, uint64_t zero_count = 0)
{
    const T time_step = s.len_aug > 1 ? end_time / T(s.len_aug - 1) : T(0);
    (void)zero_count;       // always the whole increment gradient of the batch: batch * L * d elements
    const uint64_t per = (s.L + 2) * s.d_aug;
    launch_indexed(per, (per + 1) / 2, batch, [&](auto ix, dim3 grid) {
        using I = decltype(ix);
        hipLaunchKernelGGL((increments_kernel<T, I>), grid, dim3(kBlock), 0, stream, path, inc, int64_t(batch), int64_t(length),
                           int(dimension), int(time_aug), int(lead_lag), time_step, zero_out, DivBy<I>(s.d_aug));
    });
    SIG_HIP(hipGetLastError());
}

// Everything the degree-3 matrix form needs from the device, taken before anything is launched: when the device
// cannot provide it (or rocBLAS cannot create its handle) `ok` stays false and the caller sweeps the shape instead,
// which needs B * L * d elements of workspace where this form needs up to kDeg3BufBytes more.
template <typename T>
struct Degree3Buffers {
    bool ok = false;
    uint64_t chunk = 0;     // paths per pass over the rows buffer
    T* inc = nullptr;
    T* dzinc = nullptr;     // backward only
    T* r1 = nullptr;        // backward only
    T* rows = nullptr;
    RocBlas::Handle handle = nullptr;

    void acquire(uint64_t batch, const Shape& s, hipStream_t stream, bool backward)
    {
        try {
            const uint64_t inc_elems = checked_mul(checked_mul(batch, s.L + 2, "increments"), s.d_aug, "increments");
            const uint64_t dz_elems = checked_mul(checked_mul(batch, s.L, "increments"), s.d_aug, "increments");
            const uint64_t per_path = checked_mul(checked_mul(s.L, s.d_aug * s.d_aug, "level-2 rows"), sizeof(T), "level-2 rows");
            if (per_path == 0 || per_path > kDeg3BufBytes) return;
            chunk = std::max<uint64_t>(1, std::min<uint64_t>(std::min<uint64_t>(batch, 65535), kDeg3BufBytes / per_path));
            inc = static_cast<T*>(workspace(0, checked_mul(inc_elems, sizeof(T), "increments")));
            if (backward) {
                dzinc = static_cast<T*>(workspace(1, checked_mul(dz_elems, sizeof(T), "increments")));
                r1 = static_cast<T*>(workspace(18, checked_mul(dz_elems, sizeof(T), "increments")));
            }
            rows = static_cast<T*>(workspace(19, checked_mul(chunk, per_path, "level-2 rows")));
            handle = rocblas_handle_for(stream);
            ok = true;
        } catch (const std::bad_alloc&) {
        } catch (const std::runtime_error&) {       // no rocBLAS handle
        }
    }
};

// ---------------------------------------------------------------------------
// forward  (dispatch mirrors siglib/cpsig/cp_signature.h:740-851 and
// siglib/cusig/cu_signature.cu:2592-2657)
// ---------------------------------------------------------------------------
template <typename T>
static void signature_impl(const T* path, T* out, uint64_t batch, uint64_t dimension, uint64_t length,
                           uint64_t degree, bool time_aug, bool lead_lag, T end_time, bool /*horner*/,
                           bool scalar_term, const T* correction, uint64_t correction_len)
{
    if (dimension == 0) throw std::invalid_argument("signature_cuda received path of dimension 0");
    validate_correction(correction, correction_len, dimension, degree, lead_lag);
    if (batch == 0) return;
    if (dimension > 0x3fffffff || degree > 0x7fffffff || length > (uint64_t(1) << 40))
        throw std::invalid_argument("signature_cuda: shape out of range");
    const Shape s = make_shape(dimension, length, degree, time_aug, lead_lag, scalar_term);
    check_degree_limit(s.d_aug, degree, "signature on this GPU build");
    checked_mul(checked_mul(batch, s.stride, "signature output"), sizeof(T), "signature output");
    hipStream_t stream = nullptr;
    entry_sync();   // inputs may have been produced on any stream

    // everything below runs under the workspace mutex: one flag serves all callers
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    tl_sig_nonfinite = -1;
    int* flag = nullptr;
    if (!g_stream_ordered) {
        flag = nonfinite_flag();
        *g_flag_host = 0;
    }

    const int sc = scalar_term ? 1 : 0;
    Degree3Buffers<T> d3;
    if (s.len_aug > 1 && s.d_aug > 1 && want_degree3_gemm(s.d_aug, degree, s.L, batch, sizeof(T) == 8, false) && rocblas_ready())
        d3.acquire(batch, s, stream, false);
    if (s.len_aug <= 1) {
        if (s.stride)
            hipLaunchKernelGGL((fill_trivial_kernel<T>), dim3(grid_for(batch * s.stride)), dim3(kBlock), 0, stream,
                               out, int64_t(batch), int64_t(s.stride), sc);
    } else if (degree == 0) {
        if (scalar_term)
            hipLaunchKernelGGL((fill_trivial_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out,
                               int64_t(batch), int64_t(1), 1);
    } else if (s.d_aug == 1) {
        hipLaunchKernelGGL((dim_one_fwd_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, path, out,
                           int64_t(batch), int64_t(length), int(degree), sc, flag);
    } else if (degree == 1) {
        const T time_step = end_time / T(s.len_aug - 1);
        hipLaunchKernelGGL((degree_one_fwd_kernel<T>), dim3(grid_for(batch * s.stride)), dim3(kBlock), 0, stream,
                           path, out, int64_t(batch), int64_t(length), int(dimension), int(time_aug),
                           int(lead_lag), time_step, sc, flag);
    } else if (d3.ok) {
        const int d = int(s.d_aug);
        const int64_t L = int64_t(s.L);
        const uint64_t chunk = d3.chunk;
        T* inc = d3.inc;
        T* rows = d3.rows;
        compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream);
        RocBlas::Handle h = d3.handle;
        tl_last_segments = 1;
        MainKernelTimer timer(stream, sizeof(T) == 8 ? "degree3_fwd_gemm_f64" : "degree3_fwd_gemm_f32");
        const int64_t dd = int64_t(d) * d;
        const int groups = (d + kDeg3RowsPerThread - 1) / kDeg3RowsPerThread;
        for (uint64_t first = 0; first < batch; first += chunk) {
            const int nb = int(std::min<uint64_t>(chunk, batch - first));
            const dim3 sgrid(unsigned((d + kWave - 1) / kWave), unsigned(nb), unsigned((groups + kWavesPerBlock - 1) / kWavesPerBlock));
            hipLaunchKernelGGL((degree3_fwd_scan_kernel<T>), sgrid, dim3(kBlock), 0, stream, (const T*)inc, rows, out, L, d,
                               int64_t(s.stride), sc, int64_t(first));
            // level 3 (row-major d^2 x d) = V^T Z; column-major: [d x d^2] = Z^T (stored: d x L) * (V^T stored: d^2 x L)^T
            gemm_col_major<T>(h, false, true, d, int(dd), int(L), inc + (first * (s.L + 2) + 1) * s.d_aug, d, (L + 2) * d,
                              (const T*)rows, int(dd), L * dd, T(0), out + first * s.stride + sc + d + dd, d, int64_t(s.stride), nb);
        }
        timer.stop();
        if (flag)
            hipLaunchKernelGGL((finite_rows_kernel<T>), dim3(grid_for(batch * s.stride)), dim3(kBlock), 0, stream, out,
                               int64_t(batch * s.stride), flag);
    } else if (use_degree2(false, s.d_aug, degree, batch)) {
        const int d = int(s.d_aug);
        const int tiles = (d + 15) / 16, col_groups = (tiles + kDeg2Cols - 1) / kDeg2Cols;
        const int64_t waves = int64_t(batch) * tiles * col_groups;
        // A wave walks its time range four steps per iteration, each iteration waiting for its loads: long ranges are
        // cut into slices that add into the output with atomics (d^2 atomics per slice against slice_len * d^2
        // products).  Few paths: enough slices for two waves per SIMD; otherwise slices of 256 steps.
        int64_t slices = waves * 2 <= simd_count() ? std::min<int64_t>(2 * simd_count() / waves, int64_t(s.L) / 64)
                                                   : int64_t(s.L) / 256;
        slices = std::max<int64_t>(slices, 1);
        const int64_t slice_len = ((int64_t(s.L) + slices - 1) / slices + 3) / 4 * 4;
        slices = (int64_t(s.L) + slice_len - 1) / slice_len;
        if (slices > 1)
            hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch * s.stride)), dim3(kBlock), 0, stream, out,
                               int64_t(batch * s.stride));
        const T time_step = end_time / T(s.len_aug - 1);
        // points staged through LDS: slabs of 4 * rq + 1 points by 64 channels, rq odd, at most 43 KB a slab; chunks of
        // equal length
        const size_t row_bytes = size_t(kDeg2SlabStride) * sizeof(T);
        const bool two_slabs = tiles > kWavesPerBlock;      // row and column channels of a block can differ
        const int rq_max = (sizeof(T) == 8 ? 15 : 33) / (two_slabs ? 2 : 1) | 1;
        const int64_t n_chunks = (slice_len + 4 * rq_max - 1) / (4 * rq_max);
        int rq = int((slice_len + 4 * n_chunks - 1) / (4 * n_chunks));
        rq = std::min(rq | 1, rq_max);
        const bool vec = !time_aug && !lead_lag && dimension % (16 / sizeof(T)) == 0 && reinterpret_cast<uintptr_t>(path) % 16 == 0 &&
                         4 * rq + 1 <= deg2_prefetch_rows<T>();
        // with fewer than four row tiles some of a block's waves would idle and its slabs be mostly padding (measured:
        // d = 64..256 1.4-1.5x faster staged, d <= 32 up to 3x slower)
        const bool staged = g_degree2_staged != 0 && tiles >= kWavesPerBlock;
        MainKernelTimer timer(stream, sizeof(T) == 8 ? (staged ? "degree2_fwd_f64_lds" : "degree2_fwd_f64")
                                                     : (staged ? "degree2_fwd_f32_lds" : "degree2_fwd_f32"));
        if (staged) {
            const int64_t row_groups = (tiles + kWavesPerBlock - 1) / kWavesPerBlock;
            const int64_t blocks = int64_t(batch) * row_groups * col_groups * slices;
            if (blocks > 2147483647LL) throw std::runtime_error("signature_cuda: launch too large");
            auto go = [&](auto mode) {
                hipLaunchKernelGGL((degree2_fwd_staged_kernel<T, decltype(mode)::value>), dim3(unsigned(blocks)), dim3(kBlock),
                                   size_t(4 * rq + 1) * row_bytes * (two_slabs ? 2 : 1), stream, path, out,
                                   int64_t(batch), int64_t(length), int(dimension), int(time_aug), int(lead_lag), time_step,
                                   int64_t(s.stride), sc, tiles, col_groups, int(slices), slice_len, rq,
                                   slices > 1 ? nullptr : flag);
            };
            if (vec) go(std::integral_constant<int, 2>());
            else if (!time_aug && !lead_lag) go(std::integral_constant<int, 1>());
            else go(std::integral_constant<int, 0>());
        } else {
            const int64_t total = waves * slices;
            const int64_t blocks = (total + kWavesPerBlock - 1) / kWavesPerBlock;
            if (blocks > 2147483647LL) throw std::runtime_error("signature_cuda: launch too large");
            hipLaunchKernelGGL((degree2_fwd_kernel<T>), dim3(unsigned(blocks)), dim3(kBlock), 0, stream, path, out, int64_t(batch),
                               int64_t(length), int(dimension), int(time_aug), int(lead_lag), time_step, int64_t(s.stride), sc,
                               tiles, col_groups, int(slices), slice_len, slices > 1 ? nullptr : flag);
        }
        timer.stop();
        if (slices > 1 && flag)
            hipLaunchKernelGGL((finite_rows_kernel<T>), dim3(grid_for(batch * s.stride)), dim3(kBlock), 0, stream, out,
                               int64_t(batch * s.stride), flag);
    } else if (use_deep(s.d_aug, degree)) {
        if (!deep_fits(s.d_aug, degree, batch)) throw std::runtime_error("signature_cuda: launch too large");
        const uint64_t inc_elems = checked_mul(checked_mul(batch, s.L + 2, "increments"), s.d_aug, "increments");
        T* inc = static_cast<T*>(workspace(0, checked_mul(inc_elems, sizeof(T), "increments")));
        compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream);
        FwdParams p;
        p.inc = inc; p.out = out; p.batch = int64_t(batch); p.L = int64_t(s.L); p.d = int(s.d_aug); p.out_stride = int64_t(s.stride);
        p.scalar = sc; p.stream = stream; p.nseg = 1; p.lseg = int64_t(s.L); p.nonfinite = flag;
        tl_last_segments = 1;
        MainKernelTimer timer(stream, sizeof(T) == 8 ? "deep_fwd_f64" : "deep_fwd_f32");
        SIG_HIP(launch_deep_fwd<T>(p, int(degree)));
        timer.stop();
    } else {
        const KernelEntry* e = choose_entry(false, sizeof(T) == 8, s.d_aug, degree, batch, s.L);
        if (!e)
            throw std::runtime_error("signature_cuda: no kernel for dimension " + std::to_string(s.d_aug) +
                                     ", degree " + std::to_string(degree) + " in this build");
        // Few paths cannot fill the chip with whole-path sweeps: split every path into time segments,
        // sweep all (path, segment) pairs concurrently and fold the pieces with Chen's identity.
        const TreeGeom geom = make_geom(int(s.d_aug), e->N - e->tail, e->k, e->D != 0);
        // lead-lag sweeps that skip the letters a step cannot move take the step's parity from its position in the
        // segment: segments start on even steps
        const bool sparse_ll = lead_lag && g_lead_lag_sparse != 0;
        // many channels without a compiled instance: the by-row sweep, whole paths only (its launches fill the chip).
        // Measured against the general run-time kernels (16 / 32 letters per lane) at 33 .. 96 channels, degrees 4 to 6:
        // double precision 1.0-1.46x faster; single precision 0.95-1.2x where 32 does not divide the channel count,
        // 0.72-0.89x where it does (the 32-letter kernel then has no partly empty group and feeds from two buffers).
        const bool rows_win = sizeof(T) == 8 || s.d_aug % 32 != 0;
        const bool by_rows = e->D <= 0 && rows_win && g_rows_forward != 0 && g_force_tail == 0 &&
                             rows_bwd_supported(sizeof(T), s.d_aug, degree) && rows_bwd_fits(sizeof(T), s.d_aug, degree, batch);
        int nseg = by_rows ? 1 : g_force_segments > 0
                             ? int(std::min<uint64_t>(uint64_t(g_force_segments), s.L))
                             : choose_segments(total_waves(geom, int64_t(batch)), int64_t(s.L), e->waves_per_simd(),
                                               batch * (s.full_len - 1) * sizeof(T),
                                               [&](int g) {
                                                   const double c = lane_step_cost(int(s.d_aug), e->N, e->tail, e->k) * 2.4e-9;
                                                   const bool ring = pick_variant(false, e, total_waves(geom, int64_t(batch)) * g, sparse_ll)->staged;
                                                   return ring ? c : std::max(c, 240e-9);
                                               },
                                               sizeof(T) == 8);
        const uint64_t n_coef = s.full_len - 1;
        FwdParams p;
        p.batch = int64_t(batch) * nseg; p.L = int64_t(s.L); p.d = int(s.d_aug); p.stream = stream;
        p.lseg = (int64_t(s.L) + nseg - 1) / nseg;
        if (sparse_ll) p.lseg += p.lseg & 1;
        nseg = int((int64_t(s.L) + p.lseg - 1) / p.lseg);      // drop segments the rounding left empty
        p.nseg = nseg;
        tl_last_segments = nseg;
        p.batch = int64_t(batch) * nseg;
        T* segs = nullptr;
        T* folds = nullptr;
        if (nseg == 1) {
            p.out = out; p.out_stride = int64_t(s.stride); p.scalar = sc; p.nonfinite = flag;
        } else {
            const uint64_t row_elems = checked_mul(batch, n_coef, "segment signatures");
            const uint64_t bytes = checked_mul(checked_mul(row_elems, uint64_t(nseg), "segment signatures"), sizeof(T), "segment signatures");
            segs = static_cast<T*>(workspace(2, bytes));
            // every halving step's rows, one step after the other: at most nseg + log2(nseg) rows per path
            if (nseg > 2)
                folds = static_cast<T*>(workspace(3, checked_mul(checked_mul(row_elems, uint64_t(nseg) + 32, "segment signatures"),
                                                                 sizeof(T), "segment signatures")));
            p.out = segs; p.out_stride = int64_t(n_coef); p.scalar = 0;
        }
        e = pick_variant(false, e, total_waves(geom, p.batch), sparse_ll);
        // staged sweeps of plain narrow paths form the increments themselves while staging the points
        if (!by_rows && e->staged && !time_aug && !lead_lag && e->D > 0 && e->D <= kPointFedMaxDim && g_point_fed) {
            p.inc = path;
            p.from_points = 1;
        } else {
            const uint64_t inc_elems = checked_mul(checked_mul(batch, s.L + 2, "increments"), s.d_aug, "increments");
            const uint64_t pad = uint64_t(kStageSteps + 2) * s.d_aug;    // staged sweeps read whole chunks past either end
            T* inc = static_cast<T*>(workspace(0, checked_mul(inc_elems + 2 * pad, sizeof(T), "increments"))) + pad;
            compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream);
            p.inc = inc;
        }
        const bool use_ll = !by_rows && sparse_ll && e->staged && e->fwd_lead_lag && !p.from_points;
        const std::string shown = by_rows ? std::string(sizeof(T) == 8 ? "rows_fwd_f64_n" : "rows_fwd_f32_n") + std::to_string(degree)
                                  : use_ll ? std::string(e->name) + "_ll" : std::string(e->name);
        MainKernelTimer timer(stream, shown.c_str());
        if (by_rows) SIG_HIP(launch_rows_fwd<T>(p, int(degree)));
        else SIG_HIP(use_ll ? e->fwd_lead_lag(p) : e->fwd(p));
        timer.stop(/*defer=*/true);
        if (nseg > 1) {
            // ordered product of the segment signatures by pairwise halving: ceil(log2(nseg)) launches.  An unpaired last
            // row stays where it is and joins the next step as its last row (`carry`).
            const T* src = segs;
            int src_rows = nseg;
            const T* carry = nullptr;
            int64_t carry_stride = 0;
            T* next = folds;
            for (int m = nseg; m > 1;) {
                const bool last = m == 2;
                const int pairs = m / 2;
                T* dst = last ? out : next;
                with_chen_fan(s.d_aug, [&](auto fan) {
                    constexpr int FAN = decltype(fan)::value;
                    const uint64_t items = chen_items(s.d_aug, degree, FAN);
                    launch_indexed(n_coef, items, batch * uint64_t(pairs), [&](auto ix, dim3 grid) {
                        using I = decltype(ix);
                        hipLaunchKernelGGL((chen_fold_step_kernel<T, I, FAN>), grid, dim3(kBlock), 0, stream, src, src_rows, carry,
                                           carry_stride, dst, int64_t(batch), m, last ? int64_t(s.stride) : int64_t(n_coef) * pairs,
                                           last ? sc : 0, DivBy<I>(s.d_aug), I(n_coef), I(items), last ? flag : nullptr);
                    });
                });
                SIG_HIP(hipGetLastError());
                if (m & 1) {
                    if (!carry) {       // the last row of this step's source becomes the carry
                        carry = src + uint64_t(m - 1) * n_coef;
                        carry_stride = int64_t(src_rows) * int64_t(n_coef);
                    }
                } else {
                    carry = nullptr;    // paired in this step, if there was one
                }
                src = dst;
                src_rows = pairs;
                next += batch * n_coef * uint64_t(pairs);
                m = pairs + (carry ? 1 : 0);
            }
        }
        exit_sync(stream);
        timer.read();
        if (flag) tl_sig_nonfinite = *g_flag_host;
        return;
    }
    SIG_HIP(hipGetLastError());
    exit_sync(stream);
    if (flag) tl_sig_nonfinite = *g_flag_host;
}

// ---------------------------------------------------------------------------
// backward  (siglib/cpsig/cp_signature.h:909-1019, siglib/cusig/cu_signature.cu:3417-3488)
// ---------------------------------------------------------------------------
// increment gradient -> raw path gradient; plain paths with a channel count that allows it take 16 bytes per lane
template <typename T>
static void launch_path_grad(const T* dzinc, T* out, uint64_t batch, uint64_t length, uint64_t dimension, bool time_aug,
                             bool lead_lag, hipStream_t stream, T* clear = nullptr, uint64_t clear_count = 0)
{
    constexpr int V = int(16 / sizeof(T));
    if (!time_aug && !lead_lag && dimension % V == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(dzinc) % 16 == 0) {
        const uint64_t per = length * (dimension / V);
        launch_indexed(per, per, batch, [&](auto ix, dim3 grid) {
            using I = decltype(ix);
            hipLaunchKernelGGL((path_grad_vec_kernel<T, I, V>), grid, dim3(kBlock), 0, stream, dzinc, out, int64_t(batch),
                               int64_t(length), DivBy<I>(dimension / V), clear, int64_t(clear_count));
        });
        return;
    }
    launch_indexed(length * dimension, (length * dimension + 1) / 2, batch, [&](auto ix, dim3 grid) {
        using I = decltype(ix);
        hipLaunchKernelGGL((path_grad_kernel<T, I>), grid, dim3(kBlock), 0, stream, dzinc, out, int64_t(batch),
                           int64_t(length), int(time_aug), int(lead_lag), DivBy<I>(dimension), clear, int64_t(clear_count));
    });
}

// A caller-independent block of device memory that a call carves its buffers out of instead of the workspace pool
// (the entry point that must not allocate).  With an arena the call only enqueues on `stream`: no waits, no events,
// whole-path sweeps only (a time split would need buffers of several signature sets).
struct Arena {
    char* base = nullptr;
    size_t bytes = 0, used = 0;
    hipStream_t stream = nullptr;
    void* take(size_t n)
    {
        const size_t off = (used + 255) & ~size_t(255);
        if (off > bytes || n > bytes - off)
            throw std::invalid_argument("this shape needs more than the " + std::to_string(bytes >> 20) +
                                        " MiB of built-in scratch memory; use sig_backprop_cuda_d");
        used = off + n;
        return base + off;
    }
};

template <typename T>
static void sig_backprop_impl(const T* path, T* out, const T* sig_derivs, const T* sig, uint64_t batch,
                              uint64_t dimension, uint64_t length, uint64_t degree, bool time_aug,
                              bool lead_lag, T end_time, bool scalar_term, const T* correction,
                              uint64_t correction_len, Arena* arena = nullptr)
{
    if (dimension == 0) throw std::invalid_argument("sig_backprop_cuda received path of dimension 0");
    validate_correction(correction, correction_len, dimension, degree, lead_lag);
    if (batch == 0) return;
    if (dimension > 0x3fffffff || degree > 0x7fffffff || length > (uint64_t(1) << 40))
        throw std::invalid_argument("sig_backprop_cuda: shape out of range");
    const Shape s = make_shape(dimension, length, degree, time_aug, lead_lag, scalar_term);
    check_degree_limit(s.d_aug, degree, "sig_backprop on this GPU build");
    const uint64_t out_elems = checked_mul(checked_mul(batch, length, "path gradient"), dimension, "path gradient");
    hipStream_t stream = arena ? arena->stream : nullptr;
    if (!arena) entry_sync();
    const int sc = scalar_term ? 1 : 0;
    // library buffers: the grow-only pool (under its mutex), or the caller-independent arena
    auto buffer = [&](int slot, uint64_t bytes) -> void* { return arena ? arena->take(bytes) : workspace(slot, bytes); };
    auto finish = [&] { if (!arena) exit_sync(stream); };
    std::unique_lock<std::mutex> lk(g_ws_mutex, std::defer_lock);
    auto lock_pool = [&] { if (!arena && !lk.owns_lock()) lk.lock(); };
    Degree3Buffers<T> d3;
    if (!arena && s.len_aug > 1 && want_degree3_gemm(s.d_aug, degree, s.L, batch, sizeof(T) == 8, true)) {
        lock_pool();
        if (rocblas_ready()) d3.acquire(batch, s, stream, true);
    }
    const bool degree3 = d3.ok;

    if (s.len_aug <= 1 || degree == 0) {
        if (out_elems)
            hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(out_elems)), dim3(kBlock), 0, stream, out,
                               int64_t(out_elems));
    } else if (degree == 1) {
        hipLaunchKernelGGL((degree_one_bwd_kernel<T>), dim3(grid_for(out_elems)), dim3(kBlock), 0, stream,
                           sig_derivs, out, int64_t(batch), int64_t(length), int(dimension), int(time_aug),
                           int(lead_lag), sc);
    } else if (degree3) {
        const int d = int(s.d_aug);
        const int64_t L = int64_t(s.L);
        const uint64_t dz_elems = checked_mul(checked_mul(batch, s.L, "increments"), s.d_aug, "increments");
        const uint64_t chunk = d3.chunk;
        T* inc = d3.inc;
        T* dzinc = d3.dzinc;
        T* r1 = d3.r1;
        T* rows = d3.rows;
        compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream, dzinc, dz_elems);
        hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(dz_elems)), dim3(kBlock), 0, stream, r1, int64_t(dz_elems));
        RocBlas::Handle h = d3.handle;
        MainKernelTimer timer(stream, sizeof(T) == 8 ? "degree3_bwd_gemm_f64" : "degree3_bwd_gemm_f32", true);
        const int64_t dd = int64_t(d) * d;
        const int groups = (d + kDeg3RowsPerThread - 1) / kDeg3RowsPerThread;
        for (uint64_t first = 0; first < batch; first += chunk) {
            const int nb = int(std::min<uint64_t>(chunk, batch - first));
            const T* g3 = sig_derivs + first * s.stride + sc + d + dd;
            // Y = Z G3^T
            gemm_row_major<T>(h, true, int(L), int(dd), d, inc + (first * (s.L + 2) + 1) * s.d_aug, d, (L + 2) * d, g3, d,
                              int64_t(s.stride), T(0), rows, int(dd), L * dd, nb);
            const dim3 sgrid(unsigned((d + kWave - 1) / kWave), unsigned(nb), unsigned((groups + kWavesPerBlock - 1) / kWavesPerBlock));
            hipLaunchKernelGGL((degree3_scan_kernel<T>), sgrid, dim3(kBlock), 0, stream, (const T*)inc, sig, sig_derivs, rows, dzinc, r1,
                               L, d, int64_t(s.stride), sc, int64_t(first));
            // dz += V G3
            gemm_row_major<T>(h, false, int(L), d, int(dd), (const T*)rows, int(dd), L * dd, g3, d, int64_t(s.stride), T(1),
                              dzinc + first * s.L * s.d_aug, d, L * d, nb);
        }
        hipLaunchKernelGGL((degree3_level1_kernel<T>), dim3(grid_for(batch * s.d_aug)), dim3(kBlock), 0, stream, sig_derivs, (const T*)r1,
                           dzinc, int64_t(batch), L, d, int64_t(s.stride), sc);
        timer.stop();
        launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
        SIG_HIP(hipGetLastError());
        finish();
        return;
    } else if (use_degree2(true, s.d_aug, degree, batch)) {
        lock_pool();
        const int d = int(s.d_aug);
        const uint64_t dz_elems = checked_mul(checked_mul(batch, s.L, "increments"), s.d_aug, "increments");
        T* dzinc = static_cast<T*>(buffer(1, checked_mul(dz_elems, sizeof(T), "increments")));
        T* h = static_cast<T*>(buffer(12, checked_mul(checked_mul(batch, s.d_aug, "increments"), sizeof(T), "increments")));
        const int tiles = (d + 15) / 16, col_groups = (tiles + kDeg2Cols - 1) / kDeg2Cols;
        // operands staged through LDS when a block's four waves all have 16 steps to work on and the channels fill the
        // 64-wide slabs (measured: d = 64, 256 1.6-1.75x faster staged, d = 100 equal, d <= 32 up to 2.5x slower)
        const bool staged = g_degree2_staged != 0 && tiles >= kWavesPerBlock && s.L >= 48;
        T* anti = staged ? static_cast<T*>(buffer(13, checked_mul(checked_mul(batch, s.d_aug * s.d_aug, "level-2 gradient"), sizeof(T),
                                                                  "level-2 gradient")))
                         : nullptr;
        const T time_step = end_time / T(s.len_aug - 1);
        if (g_degree2_staged != 0 && tiles >= 3 && tiles <= kDeg2Cols && s.L >= 1) {
            // at most 64 channels: one launch, the level-2 gradient's fragments in registers; plain paths receive
            // their gradient directly
            const bool plain = !time_aug && !lead_lag;
            const bool vec = plain && dimension % (16 / sizeof(T)) == 0 && reinterpret_cast<uintptr_t>(path) % 16 == 0;
            const int64_t out_rows = plain ? int64_t(s.L) + 1 : int64_t(s.L);
            const int64_t chunks = (out_rows + kDeg2BwdRows - 1) / kDeg2BwdRows;
            int64_t parts = std::min<int64_t>(chunks, std::max<int64_t>(1, (2 * int64_t(simd_count()) / 4 + int64_t(batch) - 1) / int64_t(batch)));
            const int64_t part_rows = (chunks + parts - 1) / parts * kDeg2BwdRows;
            parts = (out_rows + part_rows - 1) / part_rows;
            const int64_t blocks = int64_t(batch) * parts;
            if (blocks > 2147483647LL) throw std::runtime_error("sig_backprop_cuda: launch too large");
            MainKernelTimer timer(stream, sizeof(T) == 8 ? "degree2_bwd_f64_rows" : "degree2_bwd_f32_rows", !arena);
            auto go = [&](auto mode) {
                constexpr int MODE = decltype(mode)::value;
                if (deg2_bwd_lds_bytes<T>() > 64 * 1024)       // above the default limit of dynamic LDS
                    SIG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&degree2_bwd_rows_kernel<T, MODE>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, int(deg2_bwd_lds_bytes<T>())));
                hipLaunchKernelGGL((degree2_bwd_rows_kernel<T, MODE>), dim3(unsigned(blocks)), dim3(kBlock), deg2_bwd_lds_bytes<T>(),
                                   stream, path, sig_derivs, MODE ? out : dzinc, int64_t(batch), int64_t(length), int(dimension),
                                   int(time_aug), int(lead_lag), time_step, int64_t(s.stride), sc, int(parts), part_rows);
            };
            if (vec) go(std::integral_constant<int, 2>());
            else if (plain) go(std::integral_constant<int, 1>());
            else go(std::integral_constant<int, 0>());
            timer.stop();
            if (!plain) launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
            SIG_HIP(hipGetLastError());
            finish();
            return;
        }
        hipLaunchKernelGGL((degree2_h_kernel<T>), dim3(grid_for(batch * s.d_aug, kWavesPerBlock)), dim3(kBlock), 0, stream, path, sig_derivs, h,
                           int64_t(batch), int64_t(length), int(dimension), int(time_aug), int(lead_lag), time_step,
                           int64_t(s.stride), sc);
        if (staged && s.L >= 1 && !time_aug && !lead_lag) {
            // more than 64 channels, plain paths: accumulators of a run of rows in registers, channels walked 64 at a
            // time (with augmentation the per-element evaluation of the points makes it slower than the kernel below)
            const bool plain = true;
            const bool vec = plain && dimension % (16 / sizeof(T)) == 0 && reinterpret_cast<uintptr_t>(path) % 16 == 0;
            const int64_t out_rows = plain ? int64_t(s.L) + 1 : int64_t(s.L);
            const int64_t run = int64_t(deg2_wide_chunks<T>()) * kDeg2BwdRows;
            const int64_t parts = (out_rows + run - 1) / run;
            const int64_t blocks = int64_t(batch) * parts * col_groups;
            if (blocks > 2147483647LL) throw std::runtime_error("sig_backprop_cuda: launch too large");
            MainKernelTimer timer(stream, sizeof(T) == 8 ? "degree2_bwd_f64_wide" : "degree2_bwd_f32_wide", !arena);
            auto go = [&](auto mode) {
                constexpr int MODE = decltype(mode)::value;
                if (deg2_bwd_lds_bytes<T>() > 64 * 1024)
                    SIG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&degree2_bwd_wide_kernel<T, MODE>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, int(deg2_bwd_lds_bytes<T>())));
                hipLaunchKernelGGL((degree2_bwd_wide_kernel<T, MODE>), dim3(unsigned(blocks)), dim3(kBlock), deg2_bwd_lds_bytes<T>(),
                                   stream, path, sig_derivs, (const T*)h, MODE ? out : dzinc, int64_t(batch), int64_t(length),
                                   int(dimension), int(time_aug), int(lead_lag), time_step, int64_t(s.stride), sc, int(parts),
                                   col_groups);
            };
            if (vec) go(std::integral_constant<int, 2>());
            else if (plain) go(std::integral_constant<int, 1>());
            else go(std::integral_constant<int, 0>());
            timer.stop();
            if (!plain) launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
            SIG_HIP(hipGetLastError());
            finish();
            return;
        }
        MainKernelTimer timer(stream, sizeof(T) == 8 ? (staged ? "degree2_bwd_f64_lds" : "degree2_bwd_f64")
                                                     : (staged ? "degree2_bwd_f32_lds" : "degree2_bwd_f32"), !arena);
        if (staged) {
            hipLaunchKernelGGL((degree2_anti_kernel<T>), dim3(grid_for(batch * s.d_aug * s.d_aug)), dim3(kBlock), 0, stream,
                               sig_derivs, anti, int64_t(batch), d, int64_t(s.stride), sc);
            const int64_t time_groups = (int64_t(s.L) + kDeg2Slab - 1) / kDeg2Slab;
            const int64_t blocks = int64_t(batch) * time_groups * col_groups;
            if (blocks > 2147483647LL) throw std::runtime_error("sig_backprop_cuda: launch too large");
            const size_t lds = (size_t(kDeg2Slab) * (sizeof(T) == 8 ? 65 : 66) + size_t(kDeg2Slab) * kDeg2SlabStride) * sizeof(T);
            hipLaunchKernelGGL((degree2_bwd_staged_kernel<T>), dim3(unsigned(blocks)), dim3(kBlock), lds, stream, path,
                               (const T*)anti, (const T*)h, dzinc, int64_t(batch), int64_t(length), int(dimension), int(time_aug),
                               int(lead_lag), time_step, time_groups, col_groups);
        } else {
            const int64_t time_tiles = (int64_t(s.L) + 15) / 16;
            const int64_t total = int64_t(batch) * time_tiles * col_groups;
            const int64_t blocks = (total + kWavesPerBlock - 1) / kWavesPerBlock;
            if (blocks > 2147483647LL) throw std::runtime_error("sig_backprop_cuda: launch too large");
            hipLaunchKernelGGL((degree2_bwd_kernel<T>), dim3(unsigned(blocks)), dim3(kBlock), 0, stream, path, sig_derivs, h, dzinc,
                               int64_t(batch), int64_t(length), int(dimension), int(time_aug), int(lead_lag), time_step,
                               int64_t(s.stride), sc, time_tiles, col_groups);
        }
        timer.stop();
        launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
        SIG_HIP(hipGetLastError());
        finish();      // the workspaces stay locked until the kernels are done
        return;
    } else if (use_deep(s.d_aug, degree)) {
        if (!deep_fits(s.d_aug, degree, batch)) throw std::runtime_error("sig_backprop_cuda: launch too large");
        lock_pool();
        const uint64_t inc_elems = checked_mul(checked_mul(batch, s.L + 2, "increments"), s.d_aug, "increments");
        const uint64_t dz_elems = checked_mul(checked_mul(batch, s.L, "increments"), s.d_aug, "increments");
        T* inc = static_cast<T*>(buffer(0, checked_mul(inc_elems, sizeof(T), "increments")));
        T* dzinc = static_cast<T*>(buffer(1, checked_mul(dz_elems, sizeof(T), "increments")));
        compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream, dzinc, dz_elems);
        BwdParams p;
        p.inc = inc; p.sig = sig; p.gsig = sig_derivs; p.dzinc = dzinc; p.batch = int64_t(batch);
        p.L = int64_t(s.L); p.d = int(s.d_aug); p.sig_stride = int64_t(s.stride); p.scalar = sc; p.stream = stream;
        MainKernelTimer timer(stream, sizeof(T) == 8 ? "deep_bwd_f64" : "deep_bwd_f32", !arena);
        SIG_HIP(launch_deep_bwd<T>(p, int(degree)));
        timer.stop();
        launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
        SIG_HIP(hipGetLastError());
        finish();
        return;
    } else {
        const KernelEntry* e = choose_entry(true, sizeof(T) == 8, s.d_aug, degree, batch, s.L);
        if (!e)
            throw std::runtime_error("sig_backprop_cuda: no kernel for dimension " + std::to_string(s.d_aug) +
                                     ", degree " + std::to_string(degree) + " in this build");
        lock_pool();
        const uint64_t inc_elems = checked_mul(checked_mul(batch, s.L + 2, "increments"), s.d_aug, "increments");
        const uint64_t dz_elems = checked_mul(checked_mul(batch, s.L, "increments"), s.d_aug, "increments");
        const uint64_t dz_bytes = checked_mul(dz_elems, sizeof(T), "increments");
        const uint64_t pad = uint64_t(kStageSteps + 2) * s.d_aug;
        BwdParams p;
        p.sig = sig; p.gsig = sig_derivs; p.batch = int64_t(batch);
        p.L = int64_t(s.L); p.d = int(s.d_aug); p.sig_stride = int64_t(s.stride); p.scalar = sc; p.stream = stream;
        const TreeGeom geom = make_geom(int(s.d_aug), e->N - e->tail, e->k, e->D != 0);
        const uint64_t n_coef = s.full_len - 1;
        const KernelEntry* ef = choose_entry(false, sizeof(T) == 8, s.d_aug, degree, batch, s.L);
        // lead-lag sweeps that skip the letters a step cannot move read a step's parity off its position in the
        // segment: segments start on even steps (a lead-lag path has an even number of steps)
        const bool sparse_ll = lead_lag && g_lead_lag_sparse != 0;
        // many channels beyond the compiled table: the by-row sweep, whole paths only (its launches fill the chip)
        // (also where an instance would lose: measured at 48 .. 128 channels, degrees 3 and 4, the by-row sweep runs
        // 1.1-4x faster than compiled single-precision instances and 1-12x faster than double-precision ones; the
        // instance table leaves these backward shapes out)
        const bool rows_win = e->D <= 0 || s.d_aug >= 48;
        const bool by_rows = !arena && rows_win && g_rows_backward != 0 && g_force_tail == 0 &&
                             rows_bwd_supported(sizeof(T), s.d_aug, degree) && rows_bwd_fits(sizeof(T), s.d_aug, degree, batch);
        int nseg = (arena || by_rows || !ef || degree > uint64_t(kCombMaxLevels)) ? 1
                   : g_force_bwd_segments > 0 ? int(std::min<uint64_t>(uint64_t(g_force_bwd_segments), s.L))
                                              : choose_bwd_segments(
                                                    total_waves(geom, int64_t(batch)), int64_t(s.L), e->waves_per_simd(),
                                                    batch * n_coef * sizeof(T),
                                                    [&](int g) {
                                                        // a backward step issues about 3.2 times the forward's instructions
                                                        const double c = lane_step_cost(int(s.d_aug), e->N, e->tail, e->k) * 7.7e-9;
                                                        const bool ring = pick_variant(true, e, total_waves(geom, int64_t(batch)) * g, sparse_ll)->staged;
                                                        return ring ? c : std::max(c, 700e-9);
                                                    },
                                                    sizeof(T) == 8);
        int64_t lseg = int64_t(s.L);
        if (nseg > 1) {
            lseg = (int64_t(s.L) + nseg - 1) / nseg;
            if (sparse_ll) lseg += lseg & 1;
            nseg = int((int64_t(s.L) + lseg - 1) / lseg);
        }
        // Whole-path staged sweeps of plain narrow paths form the increments themselves while staging the points: no
        // pre-pass launch, so the accumulator comes from the pair that takes turns (cleared by the previous call).
        const KernelEntry* e_run = pick_variant(true, e, total_waves(geom, int64_t(batch) * nseg), sparse_ll);
        const bool point_fed = !arena && !by_rows && nseg == 1 && e_run->staged && !time_aug && !lead_lag && e_run->D > 0 &&
                               e_run->D <= kPointFedMaxDim && g_point_fed != 0;
        T* inc = nullptr;
        T* dzinc = nullptr;
        DzPair* turn = nullptr;
        int mine = 0;
        if (point_fed) {
            int dev = 0;
            SIG_HIP(hipGetDevice(&dev));
            turn = &g_dz[dev];
            mine = turn->next;
            dzinc = static_cast<T*>(dz_pair_buffer(*turn, mine, dz_bytes));
            if (turn->dirty[mine]) {        // first use, or a call that failed half-way: clear it here
                const uint64_t n = (turn->dirty[mine] + sizeof(T) - 1) / sizeof(T);
                hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(n)), dim3(kBlock), 0, stream, dzinc, int64_t(n));
                SIG_HIP(hipGetLastError());
                turn->dirty[mine] = 0;
            }
            p.inc = path;
            p.from_points = 1;
        } else {
            inc = static_cast<T*>(buffer(0, checked_mul(inc_elems + 2 * pad, sizeof(T), "increments"))) + pad;
            dzinc = static_cast<T*>(buffer(1, dz_bytes));
            // one launch writes the increments and clears the increment-gradient accumulator (dz_elems <= increment elements)
            compute_increments(path, inc, batch, dimension, length, time_aug, lead_lag, end_time, s, stream, dzinc, dz_elems);
            p.inc = inc;
        }
        p.dzinc = dzinc;
        if (nseg > 1) {
            // (path, segment) rows, scalar-free: segment signatures, their running products from the left (the state
            // at each segment's end), from the right (what follows each segment), and the adjoints of the states
            const uint64_t rows = checked_mul(batch, uint64_t(nseg), "segment signatures");
            const uint64_t bytes = checked_mul(checked_mul(rows, n_coef, "segment signatures"), sizeof(T), "segment signatures");
            T* segs = static_cast<T*>(buffer(2, bytes));
            T* left = static_cast<T*>(buffer(8, bytes));
            T* right = static_cast<T*>(buffer(9, bytes));
            T* adj = static_cast<T*>(buffer(10, bytes));
            const int64_t n = int64_t(n_coef);
            FwdParams f;
            f.inc = inc; f.batch = int64_t(rows); f.L = int64_t(s.L); f.d = int(s.d_aug); f.stream = stream;
            f.lseg = lseg; f.nseg = nseg; f.out = segs; f.out_stride = n; f.scalar = 0;
            const TreeGeom fgeom = make_geom(int(s.d_aug), ef->N - ef->tail, ef->k, ef->D != 0);
            ef = pick_variant(false, ef, total_waves(fgeom, f.batch), sparse_ll);
            SIG_HIP((sparse_ll && ef->staged && ef->fwd_lead_lag) ? ef->fwd_lead_lag(f) : ef->fwd(f));
            // both scans by doubling: ceil(log2(nseg)) launches, ping-ponging between two scratch copies
            int steps = 0;
            while ((1 << steps) < nseg) ++steps;
            T* scratch = steps > 1 ? static_cast<T*>(buffer(11, checked_mul(bytes, steps > 2 ? 4 : 2, "segment signatures")))
                                   : nullptr;
            const uint64_t buf = rows * n_coef;
            const T* xsrc = segs;
            const T* zsrc = segs;
            for (int k = 0; k < steps; ++k) {
                const bool last = k == steps - 1;
                T* xdst = last ? left : scratch + uint64_t(k & 1) * 2 * buf;
                T* zdst = last ? right : scratch + (uint64_t(k & 1) * 2 + 1) * buf;
                with_chen_fan(s.d_aug, [&](auto fan) {
                    constexpr int FAN = decltype(fan)::value;
                    const uint64_t items = chen_items(s.d_aug, degree, FAN);
                    launch_indexed(n_coef, items, 2 * rows, [&](auto ix, dim3 grid) {
                        using I = decltype(ix);
                        hipLaunchKernelGGL((chen_scan_step_kernel<T, I, FAN>), grid, dim3(kBlock), 0, stream, xsrc, zsrc, xdst,
                                           zdst, int64_t(batch), nseg, 1 << k, k == 0 ? 1 : 0, DivBy<I>(s.d_aug), I(n_coef),
                                           I(items));
                    });
                });
                xsrc = xdst;
                zsrc = zdst;
            }
            SIG_HIP(hipGetLastError());
            SigShape rs;
            rs.n_coef = n_coef; rs.stride = n_coef; rs.off = 0;
            SharedRows up;
            up.share = nseg; up.stride = int64_t(s.stride); up.off = sc;
            launch_combine_bwd<T>(sig_derivs, adj, nullptr, nullptr, right, rows, s.d_aug, degree, rs, stream, 1, up, 1);
            SIG_HIP(hipGetLastError());
            p.sig = left; p.gsig = adj; p.sig_stride = n; p.scalar = 0;
            p.batch = int64_t(rows); p.nseg = nseg; p.lseg = lseg;
        }
        e = e_run;
        const bool use_ll = !by_rows && sparse_ll && e->bwd_lead_lag && (s.L & 1) == 0;
        const std::string shown = by_rows ? std::string(sizeof(T) == 8 ? "rows_bwd_f64_n" : "rows_bwd_f32_n") + std::to_string(degree)
                                  : use_ll ? std::string(e->name) + "_ll" : std::string(e->name);
        MainKernelTimer timer(stream, shown.c_str(), !arena);
        if (turn) turn->dirty[mine] = dz_bytes;        // from here on the accumulator holds sums
        if (by_rows) {
            SIG_HIP(launch_rows_bwd<T>(p, int(degree)));
        } else {
            SIG_HIP(use_ll ? e->bwd_lead_lag(p) : e->bwd(p));
        }
        timer.stop();
        if (turn) {
            // the same launch clears what the other accumulator still holds: it is the next call's
            const int other = 1 - mine;
            T* clear = turn->dirty[other] ? static_cast<T*>(turn->ptr[other]) : nullptr;
            launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream, clear,
                                (turn->dirty[other] + sizeof(T) - 1) / sizeof(T));
            SIG_HIP(hipGetLastError());
            turn->dirty[other] = 0;
            turn->next = other;
        } else {
            launch_path_grad<T>(dzinc, out, batch, length, dimension, time_aug, lead_lag, stream);
            SIG_HIP(hipGetLastError());
        }
        finish();
        return;
    }
    SIG_HIP(hipGetLastError());
    finish();
}

// ---------------------------------------------------------------------------
// built-in scratch memory of the entry point that allocates nothing
// ---------------------------------------------------------------------------
constexpr size_t kScratchBytes = size_t(32) << 20;
}  // namespace sigamd

// Every GPU the library runs on holds its own copy of this array (at its own address) until the process ends.  In
// host code the name is only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
static __device__ __align__(256) unsigned char scratch[sigamd::kScratchBytes];

namespace sigamd {

static std::mutex g_scratch_mutex;
static std::map<int, void*> g_scratch_ptr;      // device -> address of that device's copy of `scratch`

static void* scratch_of_current_device()
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    auto it = g_scratch_ptr.find(dev);
    if (it != g_scratch_ptr.end()) return it->second;
    void* ptr = nullptr;
    SIG_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) throw std::runtime_error("built-in scratch memory has no device address");
    g_scratch_ptr[dev] = ptr;
    return ptr;
}

void note_alloc_retry() noexcept { ++g_alloc_retries; }

}  // namespace sigamd

using namespace sigamd;

// signature_cuda_* with the batch taken in halves when the device cannot hold the workspace of the whole call
template <typename T>
static void signature_entry(const T* path, T* out, uint64_t batch, uint64_t dimension, uint64_t length, uint64_t degree,
                            bool time_aug, bool lead_lag, T end_time, bool horner, bool scalar_term, const T* correction,
                            uint64_t correction_len)
{
    int nonfinite = 0;
    split_on_bad_alloc(batch, "signature", [&](uint64_t first, uint64_t count) {
        uint64_t stride = 0;
        if (first) stride = make_shape(dimension, length, degree, time_aug, lead_lag, scalar_term).stride;
        signature_impl<T>(path + first * length * dimension, out + first * stride, count, dimension, length, degree, time_aug,
                          lead_lag, end_time, horner, scalar_term, correction, correction_len);
        const int f = tl_sig_nonfinite;
        nonfinite = (nonfinite < 0 || f < 0) ? -1 : (nonfinite | f);
    });
    if (batch) tl_sig_nonfinite = nonfinite;
}

template <typename T>
static void sig_backprop_entry(const T* path, T* out, const T* sig_derivs, const T* sig, uint64_t batch, uint64_t dimension,
                               uint64_t length, uint64_t degree, bool time_aug, bool lead_lag, T end_time, bool scalar_term,
                               const T* correction, uint64_t correction_len)
{
    split_on_bad_alloc(batch, "sig_backprop", [&](uint64_t first, uint64_t count) {
        uint64_t stride = 0;
        if (first) stride = make_shape(dimension, length, degree, time_aug, lead_lag, scalar_term).stride;
        sig_backprop_impl<T>(path + first * length * dimension, out + first * length * dimension, sig_derivs + first * stride,
                             sig + first * stride, count, dimension, length, degree, time_aug, lead_lag, end_time, scalar_term,
                             correction, correction_len);
    });
}

extern "C" {

CUSIG_AMD_API int signature_cuda_f(const float* path, float* out, uint64_t batch_size, uint64_t dimension,
                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag, float end_time,
                                   bool horner, bool scalar_term, const float* correction,
                                   uint64_t correction_len, uint64_t, uint64_t) noexcept
{
    return guarded([&] {
        signature_entry<float>(path, out, batch_size, dimension, length, degree, time_aug, lead_lag, end_time,
                               horner, scalar_term, correction, correction_len);
    });
}

CUSIG_AMD_API int signature_cuda_d(const double* path, double* out, uint64_t batch_size, uint64_t dimension,
                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                   double end_time, bool horner, bool scalar_term, const double* correction,
                                   uint64_t correction_len, uint64_t, uint64_t) noexcept
{
    return guarded([&] {
        signature_entry<double>(path, out, batch_size, dimension, length, degree, time_aug, lead_lag, end_time,
                                horner, scalar_term, correction, correction_len);
    });
}

CUSIG_AMD_API int sig_backprop_cuda_f(const float* path, float* out, const float* sig_derivs, const float* sig,
                                      uint64_t batch_size, uint64_t dimension, uint64_t length, uint64_t degree,
                                      bool time_aug, bool lead_lag, float end_time, bool scalar_term,
                                      const float* correction, uint64_t correction_len, uint64_t,
                                      uint64_t) noexcept
{
    return guarded([&] {
        sig_backprop_entry<float>(path, out, sig_derivs, sig, batch_size, dimension, length, degree, time_aug,
                                  lead_lag, end_time, scalar_term, correction, correction_len);
    });
}

CUSIG_AMD_API int sig_backprop_cuda_d(const double* path, double* out, const double* sig_derivs,
                                      const double* sig, uint64_t batch_size, uint64_t dimension,
                                      uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                      double end_time, bool scalar_term, const double* correction,
                                      uint64_t correction_len, uint64_t, uint64_t) noexcept
{
    return guarded([&] {
        sig_backprop_entry<double>(path, out, sig_derivs, sig, batch_size, dimension, length, degree, time_aug,
                                   lead_lag, end_time, scalar_term, correction, correction_len);
    });
}

CUSIG_AMD_API int cusig_amd_sig_backprop_noalloc_d(const double* path, double* out, const double* sig_derivs,
                                                   const double* sig, uint64_t batch_size, uint64_t dimension,
                                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                                   double end_time, bool scalar_term, void* stream) noexcept
{
    return guarded([&] {
        Arena arena;
        arena.base = static_cast<char*>(scratch_of_current_device());
        arena.bytes = kScratchBytes;
        arena.stream = static_cast<hipStream_t>(stream);
        sig_backprop_impl<double>(path, out, sig_derivs, sig, batch_size, dimension, length, degree, time_aug, lead_lag,
                                  end_time, scalar_term, nullptr, 0, &arena);
    });
}

CUSIG_AMD_API uint64_t cusig_amd_noalloc_scratch_bytes(void) noexcept { return kScratchBytes; }

CUSIG_AMD_API const char* cusig_last_error_message(void) noexcept { return g_last_error; }

CUSIG_AMD_API void cusig_shutdown(void) noexcept
{
    release_workspaces();
    clear_lyndon_tables();
}

CUSIG_AMD_API uint64_t cusig_amd_sig_length(uint64_t dimension, uint64_t degree) noexcept
{
    return sig_length_u64(dimension, degree);
}

CUSIG_AMD_API void cusig_amd_set_profiling(int enabled) noexcept { g_profile = enabled != 0; }

CUSIG_AMD_API float cusig_amd_last_kernel_ms(void) noexcept { return g_last_ms; }

CUSIG_AMD_API const char* cusig_amd_last_kernel_name(void) noexcept
{
    static thread_local char name[sizeof g_last_name];
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    std::memcpy(name, g_last_name, sizeof name);
    return name;
}

CUSIG_AMD_API void cusig_amd_force_segments(int segments) noexcept { if (g_test_hooks) g_force_segments = segments; }
CUSIG_AMD_API int cusig_amd_last_segments(void) noexcept { return tl_last_segments; }
CUSIG_AMD_API void cusig_amd_set_point_fed(int on) noexcept { if (g_test_hooks) g_point_fed = on; }
CUSIG_AMD_API void cusig_amd_set_lead_lag_sparse(int on) noexcept { if (g_test_hooks) g_lead_lag_sparse = on; }

CUSIG_AMD_API void cusig_amd_force_bwd_segments(int segments) noexcept { if (g_test_hooks) g_force_bwd_segments = segments; }

CUSIG_AMD_API void cusig_amd_set_rows_backward(int on) noexcept { if (g_test_hooks) g_rows_backward = on; }
CUSIG_AMD_API void cusig_amd_set_rows_forward(int on) noexcept { if (g_test_hooks) g_rows_forward = on; }

CUSIG_AMD_API void cusig_amd_force_staged(int mode) noexcept { if (g_test_hooks) g_force_staged = mode; }

CUSIG_AMD_API void cusig_amd_force_wide_index(int enabled) noexcept { if (g_test_hooks) g_force_wide_index = enabled; }
CUSIG_AMD_API void cusig_amd_force_chen_adjoint(int mode) noexcept { if (g_test_hooks) g_chen_adjoint_mode = mode; }
CUSIG_AMD_API void cusig_amd_set_chen_low_levels(int enabled) noexcept { if (g_test_hooks) g_chen_low_levels = enabled; }

CUSIG_AMD_API void cusig_amd_set_stream_ordered(int enabled) noexcept { g_stream_ordered = enabled; }

CUSIG_AMD_API int cusig_amd_last_sig_nonfinite(void) noexcept { return tl_sig_nonfinite; }

CUSIG_AMD_API void cusig_amd_force_degree2(int mode) noexcept { if (g_test_hooks) g_force_degree2 = mode; }
CUSIG_AMD_API void cusig_amd_force_degree3(int mode) noexcept { if (g_test_hooks) g_force_degree3 = mode; }

CUSIG_AMD_API void cusig_amd_force_deep(int enabled) noexcept { if (g_test_hooks) g_force_deep = enabled; }

CUSIG_AMD_API void cusig_amd_set_degree2_staged(int enabled) noexcept { if (g_test_hooks) g_degree2_staged = enabled; }

CUSIG_AMD_API void cusig_amd_ignore_instance_table(int on) noexcept { if (g_test_hooks) g_ignore_table = on; }
CUSIG_AMD_API void cusig_amd_force_run_time_wide(int enabled) noexcept { if (g_test_hooks) g_force_run_time_wide = enabled; }

CUSIG_AMD_API void cusig_amd_force_partition(int tail, int k) noexcept
{
    if (!g_test_hooks) return;
    g_force_tail = tail;
    g_force_k = k;
}

CUSIG_AMD_API void cusig_amd_enable_test_hooks(int enabled) noexcept
{
    g_test_hooks = enabled != 0;
    if (enabled) return;
    // back to the defaults
    g_force_segments = 0;
    g_point_fed = 1;
    g_lead_lag_sparse = 1;
    g_force_bwd_segments = 0;
    g_rows_backward = 1;
    g_rows_forward = 1;
    g_force_staged = -1;
    g_force_wide_index = 0;
    g_chen_adjoint_mode = 0;
    g_chen_low_levels = 1;
    g_force_degree2 = -1;
    g_force_degree3 = -1;
    g_force_deep = 0;
    g_degree2_staged = 1;
    g_force_run_time_wide = 0;
    g_ignore_table = 0;
    g_force_tail = 0;
    g_force_k = 0;
    g_alloc_limit = 0;
}

CUSIG_AMD_API uint64_t cusig_amd_workspace_bytes(void) noexcept
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    uint64_t total = 0;
    for (const auto& kv : g_ws)
        if (kv.first.first == dev) total += kv.second.bytes;
    return total;
}

CUSIG_AMD_API void cusig_amd_set_alloc_limit(uint64_t bytes) noexcept { if (g_test_hooks) g_alloc_limit = bytes; }
CUSIG_AMD_API int cusig_amd_alloc_retries(void) noexcept { return g_alloc_retries; }

CUSIG_AMD_API int cusig_amd_kernel_choice(int backward, int is_f64, uint64_t dimension, uint64_t degree,
                                          int* tail, int* k, int* specialised) noexcept
{
    const KernelEntry* e = find_entry(backward != 0, is_f64 != 0, dimension, degree);
    if (!e) return 0;
    if (tail) *tail = e->tail;
    if (k) *k = e->k;
    if (specialised) *specialised = e->D > 0;
    return 1;
}

}  // extern "C"
