// C ABI of the gfx950 attention library: argument validation and kernel launches.
// The primary entry points only enqueue kernels on the caller's stream (no allocation, no host
// synchronisation), so they may be captured into a HIP graph.  Process-wide state kept here: the
// optional per-kernel event profiler, the cached compute-unit count and workgroup-width override, the
// per-stream scratch buffers of the reference-named backward shim (which has no workspace argument),
// and the per-device address of the static scratch of the allocation-free backward.
#include "../../include/flame_attn.h"

#include <algorithm>

#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "attn_bwd.hpp"
#include "attn_fwd.hpp"
#include "attn_fwd_bigd.hpp"
#include "prep.hpp"
#include "sage.hpp"
#include "plan_cache.hpp"
#include "tile_ops.hpp"
#include "fp8_offload.hpp"
#include "materialised.hpp"

using namespace fattn;

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// [B,H,N,D] element strides: D stride must be 1, the others multiples of 8 (16-byte rows)
int check_view(const void* base, const int64_t* st, int64_t off) {
    if (!base || !st) return FLAME_ATTN_ERR_INVALID;
    if (st[3] != 1) return FLAME_ATTN_ERR_UNSUPPORTED;
    if ((st[0] | st[1] | st[2] | off) & 7) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (st[2] >= (int64_t(1) << 24)) return FLAME_ATTN_ERR_UNSUPPORTED;   // row offsets inside a tile are kept in 32 bits
    if (st[0] < 0 || st[1] < 0 || st[2] < 0) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (!aligned16(static_cast<const uint16_t*>(base) + off)) return FLAME_ATTN_ERR_UNSUPPORTED;
    return FLAME_ATTN_OK;
}

Strides mk(const int64_t* st) { return Strides{st[0], st[1], st[2]}; }

// FLAME_ATTN_WG_WAVES=4 forces 128-query workgroups in the forward and dQ kernels (read once per process)
int wg_waves_override() {
    static const int value = [] {
        const char* v = getenv("FLAME_ATTN_WG_WAVES");
        return v ? atoi(v) : 8;
    }();
    return value;
}


// Optional per-kernel timing with HIP events on the caller's stream (off by default; when off the
// launch path touches none of this).  Event pairs are created on demand and summed on read.
struct Profiler {
    static constexpr int kKinds = FLAME_ATTN_N_KERNEL_KINDS;
    static constexpr size_t kMaxPairs = 8192;
    std::mutex mu;
    std::atomic<bool> enabled{false};     // read without the lock on every launch
    std::vector<hipEvent_t> start[kKinds], stop[kKinds];
    size_t used[kKinds] = {};

    hipEvent_t begin(int kind, hipStream_t s, size_t* slot) {
        std::lock_guard<std::mutex> g(mu);
        if (!enabled.load(std::memory_order_relaxed) || used[kind] >= kMaxPairs) return nullptr;
        if (used[kind] == start[kind].size()) {
            hipEvent_t a, b;
            if (hipEventCreate(&a) != hipSuccess) return nullptr;
            if (hipEventCreate(&b) != hipSuccess) { (void)hipEventDestroy(a); return nullptr; }
            start[kind].push_back(a);
            stop[kind].push_back(b);
        }
        *slot = used[kind]++;
        (void)hipEventRecord(start[kind][*slot], s);
        return stop[kind][*slot];
    }
};
Profiler g_prof;
#ifdef FLAME_ATTN_PHASE_TIMING
unsigned long long* g_phase_cycles = nullptr;   // device buffer set by flame_attn_debug_set_phase_buffer
#endif

struct ScopedKernelTimer {
    hipEvent_t stop_ev = nullptr;
    hipStream_t s;
    ScopedKernelTimer(int kind, hipStream_t stream) : s(stream) {
        if (g_prof.enabled.load(std::memory_order_relaxed)) {
            size_t slot;
            stop_ev = g_prof.begin(kind, stream, &slot);
        }
    }
    ~ScopedKernelTimer() {
        if (stop_ev) (void)hipEventRecord(stop_ev, s);
    }
};

template <int D, bool HASMASK, int NW, bool VECMASK = false>
int launch_fwd(const FwdParams& p, hipStream_t s) {
    using T = FwdTile<D>;
    constexpr int BM = 32 * NW;
    static bool attr_done = false;   // idempotent, so a benign race at worst repeats the call
    auto kern = fwd_kernel<D, HASMASK, NW, VECMASK>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    const int64_t n_qt = (p.Sq + BM - 1) / BM;
    const int64_t grid = n_qt * p.B * p.H;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_FWD, s);
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * NW), T::LDS_BYTES, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

// 256-query workgroups, one wavefront per SIMD (builds without keep-mask / bias only)
template <int D>
int launch_fwd_wide(const FwdParams& p, hipStream_t s) {
    using T = FwdWideTile<D>;
    static bool attr_done = false;
    auto kern = fwd_wide_kernel<D>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    const int64_t n_qt = (p.Sq + T::BM - 1) / T::BM;
    const int64_t grid = n_qt * p.B * p.H;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_FWD, s);
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), T::LDS_BYTES, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// FLAME_ATTN_BWD_SCHEDULE selects how the backward of a problem with equally long walks is launched (read at every
// call, so that one process can time the variants against each other):
//   unset / anything else  dQ kernel (which also forms the per-query rows), then dK/dV kernel     [the default]
//   "joint"                per-query rows by a pass of their own, then dQ and dK/dV workgroups in one grid
//   "rows"                 per-query rows by a pass of their own, then the two kernels one after the other
// Measured at B=1 H=24 S=4608 D=128: the joint grid is 0.8 % faster than the default, within the spread between
// machines; it stays selectable so that the comparison can be repeated.
int bwd_schedule_override() {
    const char* v = getenv("FLAME_ATTN_BWD_SCHEDULE");
    if (!v) return 0;
    return strcmp(v, "joint") == 0 ? 1 : strcmp(v, "rows") == 0 ? 2 : 0;
}

// Head dims: the kernels are compiled for 64 and 128; any other multiple of 8 up to 128 (96 among them) runs
// zero-padded on the next compiled size.
bool head_dim_ok(int D) { return D > 0 && D <= 128 && D % 8 == 0; }
// head dims served by the forward alone, in chunks of 128 (attn_fwd_bigd.hpp)
bool big_head_dim_ok(int D) { return D > 128 && D <= 512 && D % 8 == 0; }
int padded_head_dim(int D) { return D <= 64 ? 64 : 128; }

// compute units of the current device (cached; 256 when the query fails)
int device_cu_count() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cus = n;
        else
            cus = 256;
    }
    return cus;
}

// backward workspace: [-delta rows][lse2 rows][fp32 partials of the split dK/dV workgroups]
size_t bwd_rows_bytes(int B, int H, int N_q) { return 2 * align_up((size_t)B * H * N_q * sizeof(float), 256); }
size_t bwd_split_slot_bytes(int D) { return (size_t)2 * 128 * D * sizeof(float); }   // dK^T and dV^T of one 128-key block

template <int D, bool HASMASK, bool TIMING = false>
int launch_bwd(const BwdParams& p, hipStream_t s) {
    using T = BwdTile<D>;
    using TQ = BwdDqTile<D>;
    static bool attr_done = false;
    auto kern = bwd_dkdv_kernel<D, HASMASK, TIMING>;
    auto kern_dq = bwd_dq_kernel<D, HASMASK, 4>;
    auto kern_dqv = bwd_dq_kernel<D, true, 4, true>;                 // keep-mask with vector-loadable rows over whole tiles
    auto kern_kvv = bwd_dkdv_kernel<D, true, false, true>;           // ... whose tiles travel through LDS
    using TW = BwdDqWideTile<D>;
    auto kern_dqw = bwd_dq_wide_kernel<D>;                           // 256-query workgroups, builds without a keep-mask only
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_dq),
                                hipFuncAttributeMaxDynamicSharedMemorySize, TQ::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_dqw),
                                hipFuncAttributeMaxDynamicSharedMemorySize, TW::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        if (HASMASK) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_dqv),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, TQ::LDS_BYTES);
            if (e != hipSuccess) return (int)e;
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_kvv),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES_VECMASK);
            if (e != hipSuccess) return (int)e;
        }
        attr_done = true;
    }
    const int64_t n_kt = (p.Sk + T::BN - 1) / T::BN;
    const int64_t grid = n_kt * p.B * p.H;
    // 256-query workgroups (4 wavefronts of 64 queries) when they neither add padding rows nor leave compute units idle
    const int64_t n256 = (p.Sq + 255) / 256;
    // (with key lengths the walks differ in length and the longest ones set the time: unless the units fill two
    // rounds, twice as many workgroups of half the size finish sooner)
    const bool wide = !HASMASK && n256 * 256 <= ((int64_t)(p.Sq + 127) / 128) * 128 && n256 * p.B * p.H >= device_cu_count() &&
                      !(p.m.kv_len && n256 * p.B * p.H < 2 * device_cu_count()) && wg_waves_override() != 4;
    const int64_t n_qt = wide ? n256 : (p.Sq + TQ::BM - 1) / TQ::BM;
    const int64_t grid_dq = n_qt * p.B * p.H;
    if (grid > 0x7fffffff || grid_dq > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    // Equally long walks everywhere and 256-query workgroups: a pass over O and dO leaves the per-query rows in the
    // workspace, then dQ and dK/dV workgroups share one grid (bwd_joint_kernel).
    const int joint_mode = bwd_schedule_override();
    if (joint_mode != 0 && wide && !HASMASK && !TIMING && !p.m.causal && !p.m.kv_len && p.split_ws) {
        static bool joint_attr_done = false;
        auto kern_joint = bwd_joint_kernel<D>;
        if (!joint_attr_done) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_joint), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               std::max(T::LDS_BYTES, TW::LDS_BYTES));
            if (e != hipSuccess) return (int)e;
            joint_attr_done = true;
        }
        BwdParams pj = p;
        pj.rows_ready = 1;
        const int64_t n_rows = (int64_t)p.B * p.H * p.Sq;
        constexpr int rows_per_wg = 256 / (D / 8);
        {
            ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_ROWS, s);
            hipLaunchKernelGGL(bwd_rows_kernel<D>, dim3((unsigned)((n_rows + rows_per_wg - 1) / rows_per_wg)), dim3(256), 0, s, pj);
        }
        const int cus = device_cu_count();
        const size_t room = p.split_ws_bytes / bwd_split_slot_bytes(D);
        // the key blocks of the last partial round are cut in two along the walk, as in the default schedule
        int64_t n_split_j = grid % cus;
        int parts = 2;
        while (parts > 1 && (size_t)(n_split_j * parts) > room) --parts;
        if (parts == 1 || (p.Sq + T::BM - 1) / T::BM < 16) n_split_j = 0;
        if (n_split_j > 0) {
            pj.n_whole = (int)(grid - n_split_j);
            pj.split_parts = parts;
        }
        const int64_t grid_kv_j = n_split_j > 0 ? pj.n_whole + n_split_j * parts : grid;
        if (joint_mode == 1) {
            pj.joint_n_dq = (int)grid_dq;
            if (grid_dq + grid_kv_j > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
            ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_JOINT, s);
            hipLaunchKernelGGL(kern_joint, dim3((unsigned)(grid_dq + grid_kv_j)), dim3(256), std::max(T::LDS_BYTES, TW::LDS_BYTES), s, pj);
        } else {      // the same kernels one after the other, reading the rows of the pre-pass
            {
                ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DQ, s);
                hipLaunchKernelGGL(kern_dqw, dim3((unsigned)grid_dq), dim3(256), TW::LDS_BYTES, s, pj);
            }
            ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DKDV, s);
            hipLaunchKernelGGL(kern, dim3((unsigned)grid_kv_j), dim3(256), T::LDS_BYTES, s, pj);
        }
        if (n_split_j > 0) {
            ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_MERGE, s);
            hipLaunchKernelGGL(bwd_dkdv_merge_kernel<D>, dim3((unsigned)(n_split_j * (D / 32))), dim3(256), 0, s, pj);
        }
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
    }
    // dQ first: besides dQ it leaves -delta = -rowsum(dO * O) and the rescaled LSE of every query row in the
    // workspace, which the dK/dV kernel stages per query tile.
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DQ, s);
        if (wide) hipLaunchKernelGGL(kern_dqw, dim3((unsigned)grid_dq), dim3(256), TW::LDS_BYTES, s, p);
        else if (HASMASK && p.m.rows16 && p.Sk % TQ::BN == 0) hipLaunchKernelGGL(kern_dqv, dim3((unsigned)grid_dq), dim3(256), TQ::LDS_BYTES, s, p);
        else hipLaunchKernelGGL(kern_dq, dim3((unsigned)grid_dq), dim3(256), TQ::LDS_BYTES, s, p);
    }
    // The dK/dV kernel keeps one workgroup per compute unit.  When the key blocks do not fill the last
    // round of that schedule, the blocks of the last round are split over the idle units along the query
    // walk (fp32 partial sums, merged by a small second kernel).  Needs equally long walks (no causal,
    // key-length or explicit mask) and room in the workspace.
    BwdParams pk = p;
    int64_t grid_kv = grid;
    int n_split = 0;
    {
        const int cus = device_cu_count();
        const int64_t rem = grid % cus;
        const int64_t n_qtiles = (p.Sq + T::BM - 1) / T::BM;
        const bool uniform = !HASMASK && !p.m.causal && !p.m.kv_len;
        if (uniform && grid > cus && rem > 0 && 2 * rem <= cus && n_qtiles >= 16 && p.split_ws) {
            int parts = (int)std::min<int64_t>(cus / rem, 4);
            const size_t room = p.split_ws_bytes / bwd_split_slot_bytes(D);
            while (parts > 1 && (size_t)(rem * parts) > room) --parts;
            if (parts > 1) {
                pk.n_whole = (int)(grid - rem);
                pk.split_parts = parts;
                n_split = (int)rem;
                grid_kv = pk.n_whole + rem * parts;
            }
        }
    }
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DKDV, s);
        if (HASMASK && !TIMING && p.m.rows16 && !p.m.causal && p.Sk % T::BN == 0 && p.Sq % T::BM == 0 &&
            (int64_t)T::BM * p.m.sq < (int64_t)1 << 31)
            hipLaunchKernelGGL(kern_kvv, dim3((unsigned)grid_kv), dim3(256), T::LDS_BYTES_VECMASK, s, pk);
        else
            hipLaunchKernelGGL(kern, dim3((unsigned)grid_kv), dim3(256), T::LDS_BYTES, s, pk);
    }
    if (n_split > 0) {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_MERGE, s);
        hipLaunchKernelGGL(bwd_dkdv_merge_kernel<D>, dim3((unsigned)(n_split * (D / 32))), dim3(256), 0, s, pk);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int lib_scratch_get(size_t need, hipStream_t stream, void** out);
std::mutex& lib_scratch_enqueue_mutex();

// Where the key-split forward for head dims above 128 may put its fp32 partial outputs.
struct FwdScratch {
    void* ws = nullptr;          // caller workspace (device memory, 16-byte aligned), or null
    size_t bytes = 0;
    bool library = false;        // reference-named entry points only: the library's own per-(device, stream) buffer
};

// Workgroups that share one query tile of the big-head-dim forward, each over a slice of the key tiles: more than one
// only where the query tiles alone leave at least half of the 256 compute units idle, at most 8, never above 256
// workgroups in all, and at least 8 key tiles (256 keys) per slice.
inline int bigd_key_splits(int64_t query_tile_wgs, int Sk) {
    if (query_tile_wgs <= 0 || query_tile_wgs * 2 > 256) return 1;
    int ks = (int)std::min<int64_t>(8, 256 / query_tile_wgs);
    ks = std::min(ks, (Sk + 31) / 32 / 8);
    return std::max(ks, 1);
}

// queries per workgroup of the big-head-dim forward the library launches for head dim D
inline int bigd_query_tile(int D) { return D <= 256 ? 128 : 64; }
inline size_t bigd_partials_bytes(int key_splits, int64_t rows, int dv) { return (size_t)key_splits * rows * (dv + 1) * sizeof(float); }

template <int NC, int NW>
int launch_fwd_bigd_nw(const FwdParams& fp, hipStream_t s, const FwdScratch& sc) {
    constexpr bool SPLIT = NC > 2;
    using T = FwdBigDTile<NC, SPLIT, NW>;
    static bool attr_done = false;
    auto kern = fwd_bigd_kernel<NC, SPLIT, NW>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    FwdBigDParams p;
    static_cast<FwdParams&>(p) = fp;
    const int64_t grid0 = (int64_t)((p.Sq + T::BM - 1) / T::BM) * p.B * p.H;
    p.key_splits = bigd_key_splits(grid0, p.Sk);
    p.part_o = nullptr;
    p.part_lse = nullptr;
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    static_assert(T::BM == (NC <= 2 ? 128 : 64), "bigd_query_tile must name this kernel's query tile");
    std::unique_lock<std::mutex> enqueue(lib_scratch_enqueue_mutex(), std::defer_lock);
    if (p.key_splits > 1) {
        // partial outputs (at most 256 workgroups x 128 queries x (512 + 1) floats = 67 MB): the caller's workspace,
        // with as many slices as fit into it; without one the keys are not split (nothing is allocated here), except
        // behind the reference-named entry points, which take the library's per-(device, stream) buffer
        void* ws = nullptr;
        if (sc.ws && aligned16(sc.ws)) {
            while (p.key_splits > 1 && bigd_partials_bytes(p.key_splits, rows, p.dv) > sc.bytes) --p.key_splits;
            ws = sc.ws;
        } else if (sc.library) {
            enqueue.lock();          // held until both kernels are enqueued
            const int rc = lib_scratch_get(bigd_partials_bytes(p.key_splits, rows, p.dv), s, &ws);
            if (rc == FLAME_ATTN_ERR_UNSUPPORTED) p.key_splits = 1;      // under a capture and nothing allocated yet: unsplit
            else if (rc) return rc;
        } else {
            p.key_splits = 1;
        }
        if (p.key_splits > 1) {
            p.part_o = static_cast<float*>(ws);
            p.part_lse = p.part_o + (size_t)p.key_splits * rows * p.dv;
        }
    }
    const int64_t grid = grid0 * p.key_splits;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_FWD, s);
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * NW), T::LDS_BYTES, s, p);
        if (p.key_splits > 1) {
            const int64_t lanes = rows * (p.dv / 4);
            hipLaunchKernelGGL(fwd_bigd_merge_kernel, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, s, p);
        }
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}
template <int NC>
int launch_fwd_bigd(const FwdParams& p, hipStream_t s, const FwdScratch& sc) { return launch_fwd_bigd_nw<NC, 4>(p, s, sc); }

// Dropout of the probabilities: the 128-query forward and dQ kernels and the dK/dV kernel in their DROPOUT
// instantiations, without the split of the last round; HASMASK: the general kernels for an explicit mask or bias.
template <int D, bool HASMASK>
int launch_fwd_dropout(const FwdParams& p, hipStream_t s) {
    using T = FwdTile<D>;
    static bool attr_done = false;
    auto kern = fwd_kernel<D, HASMASK, 4, false, true>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    const int64_t grid = (int64_t)((p.Sq + 127) / 128) * p.B * p.H;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_FWD, s);
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), T::LDS_BYTES, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

template <int D, bool HASMASK>
int launch_bwd_dropout(const BwdParams& p, hipStream_t s) {
    using T = BwdTile<D>;
    using TQ = BwdDqTile<D>;
    static bool attr_done = false;
    auto kern = bwd_dkdv_kernel<D, HASMASK, false, false, true>;
    auto kern_dq = bwd_dq_kernel<D, HASMASK, 4, false, true>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_dq),
                                hipFuncAttributeMaxDynamicSharedMemorySize, TQ::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    const int64_t grid = (int64_t)((p.Sk + T::BN - 1) / T::BN) * p.B * p.H;
    const int64_t grid_dq = (int64_t)((p.Sq + TQ::BM - 1) / TQ::BM) * p.B * p.H;
    if (grid > 0x7fffffff || grid_dq > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DQ, s);        // first: it leaves -delta and the rescaled LSE rows
        hipLaunchKernelGGL(kern_dq, dim3((unsigned)grid_dq), dim3(256), TQ::LDS_BYTES, s, p);
    }
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_BWD_DKDV, s);
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), T::LDS_BYTES, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

// 0 <= p < 1 (src/autograd_v4/ops/sdpa.rs:110-116); fills the kernel-side description of the draw
// draw_cq / draw_ck: the tiles of the reference's chunked draw (0, or at least the sequence: the whole axis)
bool set_dropout(MaskArgs& m, float dropout_p, uint64_t dropout_seed, int draw_cq, int draw_ck, int Sq, int Sk) {
    if (!(dropout_p >= 0.f) || !(dropout_p < 1.f) || draw_cq < 0 || draw_ck < 0) return false;
    const int cq = (draw_cq == 0 || draw_cq > Sq) ? Sq : draw_cq, ck = (draw_ck == 0 || draw_ck > Sk) ? Sk : draw_ck;
    m.drop_cq = (cq == Sq && ck == Sk) ? 0u : (uint32_t)cq;
    m.drop_ck = (uint32_t)ck;
    m.drop_seed = (uint32_t)dropout_seed;
    m.drop_thr = (uint32_t)ceil((double)dropout_p * 16777216.0);      // u >= p  <=>  24-bit integer >= ceil(p * 2^24)
    const float keep = 1.0f - dropout_p;
    m.drop_scale = 1.0f / keep;
    return true;
}

}  // namespace

extern "C" {

#ifdef FLAME_ATTN_PHASE_TIMING
// Development builds only: device buffer of 6 uint64 per workgroup that the timing build of the dK/dV
// kernel fills with per-phase cycle counts (null switches it off again).
int flame_attn_debug_set_phase_buffer(void* device_buffer) {
    g_phase_cycles = static_cast<unsigned long long*>(device_buffer);
    return FLAME_ATTN_OK;
}
#endif

int flame_attn_profiling_enable(int on) {
    std::lock_guard<std::mutex> g(g_prof.mu);
    g_prof.enabled.store(on != 0, std::memory_order_relaxed);
    for (int k = 0; k < Profiler::kKinds; ++k) g_prof.used[k] = 0;
    return FLAME_ATTN_OK;
}

int flame_attn_profiling_read(FlameAttnKernelTimes* out) {
    if (!out) return FLAME_ATTN_ERR_INVALID;
    std::lock_guard<std::mutex> g(g_prof.mu);
    for (int k = 0; k < Profiler::kKinds; ++k) {
        double total = 0.0;
        for (size_t i = 0; i < g_prof.used[k]; ++i) {
            hipError_t e = hipEventSynchronize(g_prof.stop[k][i]);
            if (e != hipSuccess) return (int)e;
            float ms = 0.f;
            e = hipEventElapsedTime(&ms, g_prof.start[k][i], g_prof.stop[k][i]);
            if (e != hipSuccess) return (int)e;
            total += ms;
        }
        out->total_ms[k] = total;
        out->launches[k] = (int)g_prof.used[k];
        g_prof.used[k] = 0;
    }
    return FLAME_ATTN_OK;
}

size_t flame_attn_bwd_workspace_bytes(int B, int H, int N_q, int D) {
    if (B <= 0 || H <= 0 || N_q <= 0 || D <= 0) return 0;
    return bwd_rows_bytes(B, H, N_q) + (size_t)device_cu_count() * bwd_split_slot_bytes(padded_head_dim(D));
}

static int attn_bwd_impl(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                        const void* LSE, void* dQ, void* dK, void* dV,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                        const int64_t* dk_strides, const int64_t* dv_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                        int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* workspace, size_t workspace_bytes, void* stream, float dropout_p, uint64_t dropout_seed,
                        int draw_cq = 0, int draw_ck = 0) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return FLAME_ATTN_ERR_INVALID;
    if (!(scale > 0.f) || !isfinite(scale)) return FLAME_ATTN_ERR_INVALID;
    if (!LSE || !workspace) return FLAME_ATTN_ERR_INVALID;
    if (!head_dim_ok(D)) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (workspace_bytes < bwd_rows_bytes(B, H, N_q)) return FLAME_ATTN_ERR_INVALID;
    if (!aligned16(workspace)) return FLAME_ATTN_ERR_UNSUPPORTED;
    int rc;
    if ((rc = check_view(Q, q_strides, q_off))) return rc;
    if ((rc = check_view(K, k_strides, k_off))) return rc;
    if ((rc = check_view(V, v_strides, v_off))) return rc;
    if ((rc = check_view(O, o_strides, o_off))) return rc;
    if ((rc = check_view(dO, do_strides, do_off))) return rc;
    if ((rc = check_view(dQ, dq_strides, dq_off))) return rc;
    if ((rc = check_view(dK, dk_strides, dk_off))) return rc;
    if ((rc = check_view(dV, dv_strides, dv_off))) return rc;
    if (keep_mask && !mask_strides) return FLAME_ATTN_ERR_INVALID;

    BwdParams p;
    p.q = static_cast<const uint16_t*>(Q) + q_off;
    p.k = static_cast<const uint16_t*>(K) + k_off;
    p.v = static_cast<const uint16_t*>(V) + v_off;
    p.o = static_cast<const uint16_t*>(O) + o_off;
    p.dout = static_cast<const uint16_t*>(dO) + do_off;
    p.lse = static_cast<const float*>(LSE) + lse_off;
    p.dq = static_cast<uint16_t*>(dQ) + dq_off;
    p.dk = static_cast<uint16_t*>(dK) + dk_off;
    p.dv = static_cast<uint16_t*>(dV) + dv_off;
    const size_t rows = (size_t)B * H * N_q;
    p.ndelta = static_cast<float*>(workspace);
    p.lse2 = reinterpret_cast<float*>(static_cast<char*>(workspace) + align_up(rows * sizeof(float), 256));
    p.split_ws = reinterpret_cast<float*>(static_cast<char*>(workspace) + bwd_rows_bytes(B, H, N_q));
    p.split_ws_bytes = workspace_bytes - bwd_rows_bytes(B, H, N_q);
    p.qs = mk(q_strides); p.ks = mk(k_strides); p.vs = mk(v_strides); p.os = mk(o_strides);
    p.dos = mk(do_strides); p.dqs = mk(dq_strides); p.dks = mk(dk_strides); p.dvs = mk(dv_strides);
    p.B = B; p.H = H; p.Sq = N_q; p.Sk = N_kv;
    p.d = D;
    p.scale = scale;
    p.m.kv_len = kv_len;
    p.m.mask = keep_mask;
    p.m.sb = keep_mask ? mask_strides[0] : 0;
    p.m.sh = keep_mask ? mask_strides[1] : 0;
    p.m.sq = keep_mask ? mask_strides[2] : 0;
    p.m.sk = keep_mask ? mask_strides[3] : 0;
    p.m.rows16 = keep_mask && p.m.sk == 1 && (reinterpret_cast<uintptr_t>(keep_mask) | (uintptr_t)p.m.sb | (uintptr_t)p.m.sh |
                                              (uintptr_t)p.m.sq) % 16 == 0;
    p.m.causal = causal ? 1 : 0;
    p.phase_cycles = nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
#ifdef FLAME_ATTN_PHASE_TIMING
    p.phase_cycles = g_phase_cycles;
    if (D == 128 && !keep_mask && g_phase_cycles) return launch_bwd<128, false, true>(p, s);   // phase-timing build
#endif
    if (dropout_p != 0.f) {
        if (!set_dropout(p.m, dropout_p, dropout_seed, draw_cq, draw_ck, N_q, N_kv)) return FLAME_ATTN_ERR_INVALID;
        if (padded_head_dim(D) == 128) return keep_mask ? launch_bwd_dropout<128, true>(p, s) : launch_bwd_dropout<128, false>(p, s);
        return keep_mask ? launch_bwd_dropout<64, true>(p, s) : launch_bwd_dropout<64, false>(p, s);
    }
    if (padded_head_dim(D) == 128) return keep_mask ? launch_bwd<128, true>(p, s) : launch_bwd<128, false>(p, s);
    return keep_mask ? launch_bwd<64, true>(p, s) : launch_bwd<64, false>(p, s);
}

int flame_attn_bwd_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                        const void* LSE, void* dQ, void* dK, void* dV,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                        const int64_t* dk_strides, const int64_t* dv_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                        int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* workspace, size_t workspace_bytes, void* stream) {
    return attn_bwd_impl(Q, K, V, O, dO, LSE, dQ, dK, dV, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         do_strides, dq_strides, dk_strides, dv_strides, q_off, k_off, v_off, o_off, do_off, lse_off, dq_off,
                         dk_off, dv_off, causal, kv_len, keep_mask, mask_strides, workspace, workspace_bytes, stream, 0.f, 0);
}

int flame_attn_bwd_dropout_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                const void* LSE, void* dQ, void* dK, void* dV,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                const int64_t* dk_strides, const int64_t* dv_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                float dropout_p, uint64_t dropout_seed,
                                void* workspace, size_t workspace_bytes, void* stream) {
    return attn_bwd_impl(Q, K, V, O, dO, LSE, dQ, dK, dV, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         do_strides, dq_strides, dk_strides, dv_strides, q_off, k_off, v_off, o_off, do_off, lse_off, dq_off,
                         dk_off, dv_off, causal, kv_len, keep_mask, mask_strides, workspace, workspace_bytes, stream, dropout_p,
                         dropout_seed);
}

int flame_attn_bwd_dropout_tiled_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                      const void* LSE, void* dQ, void* dK, void* dV,
                                      int B, int H, int N_q, int N_kv, int D, float scale,
                                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                      const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                      const int64_t* dk_strides, const int64_t* dv_strides,
                                      int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                      int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                      int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                      float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                      void* workspace, size_t workspace_bytes, void* stream) {
    return attn_bwd_impl(Q, K, V, O, dO, LSE, dQ, dK, dV, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         do_strides, dq_strides, dk_strides, dv_strides, q_off, k_off, v_off, o_off, do_off, lse_off, dq_off,
                         dk_off, dv_off, causal, kv_len, keep_mask, mask_strides, workspace, workspace_bytes, stream, dropout_p,
                         dropout_seed, draw_chunk_q, draw_chunk_kv);
}

int flame_sage_quant_qk_int8(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                             const int64_t* q_strides, const int64_t* k_strides, int64_t q_off, int64_t k_off,
                             int smooth_k, void* Qi8, void* Ki8, void* q_scales, void* k_scales, void* k_mean,
                             void* stream) {
    return flame_sage_quant_qk_int8_ks(Q, K, B, H, N_q, N_kv, D, q_strides, k_strides, q_off, k_off, smooth_k, Qi8, Ki8,
                                       q_scales, k_scales, k_mean, nullptr, stream);
}

int flame_sage_quant_qk_int8_ks(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                                const int64_t* q_strides, const int64_t* k_strides, int64_t q_off, int64_t k_off,
                                int smooth_k, void* Qi8, void* Ki8, void* q_scales, void* k_scales, void* k_mean,
                                void* K_smoothed, void* stream) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return FLAME_ATTN_ERR_INVALID;
    if (K_smoothed && !aligned16(K_smoothed)) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (!Qi8 || !Ki8 || !q_scales || !k_scales || !k_mean) return FLAME_ATTN_ERR_INVALID;
    if (!head_dim_ok(D)) return FLAME_ATTN_ERR_UNSUPPORTED;
    const int Dp = padded_head_dim(D);      // row length of everything written here (flame_sage_row_elems)
    int rc;
    if ((rc = check_view(Q, q_strides, q_off))) return rc;
    if ((rc = check_view(K, k_strides, k_off))) return rc;
    if (!aligned16(Qi8) || !aligned16(Ki8) || !aligned16(k_mean)) return FLAME_ATTN_ERR_UNSUPPORTED;
    SageQuantParams p;
    p.d = D;
    p.q = static_cast<const uint16_t*>(Q) + q_off;
    p.k = static_cast<const uint16_t*>(K) + k_off;
    p.qs = mk(q_strides); p.ks = mk(k_strides);
    p.B = B; p.H = H; p.Sq = N_q; p.Sk = N_kv;
    p.smooth_k = smooth_k ? 1 : 0;
    p.kmean = static_cast<float*>(k_mean);
    p.qi8 = static_cast<int8_t*>(Qi8);
    p.ki8 = static_cast<int8_t*>(Ki8);
    p.sq = static_cast<float*>(q_scales);
    p.sk = static_cast<float*>(k_scales);
    p.ks_out = static_cast<uint16_t*>(K_smoothed);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t bh = (int64_t)B * H;
    // workgroups per (batch, head): one per Q block, one per pair of K blocks
    const int64_t nblk = (N_q + kSageQBlk - 1) / kSageQBlk + ((N_kv + kSageKBlk - 1) / kSageKBlk + 1) / 2;
    if (bh * nblk > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_SAGE_KMEAN, s);
        // the partial sums of a head (n_chunks * D doubles) must fit in that head's int8 K output
        const int n_chunks = (int)std::max<int64_t>(1, std::min<int64_t>(32, N_kv / 256));
        const int rows_per_chunk = (N_kv + n_chunks - 1) / n_chunks;
        if (N_kv < 256) {       // short: one workgroup per head sums all rows
            if (Dp == 128) hipLaunchKernelGGL(sage_kmean_kernel<128>, dim3((unsigned)bh), dim3(512), 0, s, p);
            else hipLaunchKernelGGL(sage_kmean_kernel<64>, dim3((unsigned)bh), dim3(512), 0, s, p);
        } else {
        if (smooth_k) {
            if (Dp == 128) hipLaunchKernelGGL(sage_kmean_partial_kernel<128>, dim3((unsigned)(bh * n_chunks)), dim3(512), 0, s, p, n_chunks, rows_per_chunk);
            else hipLaunchKernelGGL(sage_kmean_partial_kernel<64>, dim3((unsigned)(bh * n_chunks)), dim3(512), 0, s, p, n_chunks, rows_per_chunk);
        }
        if (Dp == 128) hipLaunchKernelGGL(sage_kmean_final_kernel<128>, dim3((unsigned)bh), dim3(128), 0, s, p, n_chunks);
        else hipLaunchKernelGGL(sage_kmean_final_kernel<64>, dim3((unsigned)bh), dim3(64), 0, s, p, n_chunks);
        }
    }
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_SAGE_QUANT, s);
        if (Dp == 128) hipLaunchKernelGGL(sage_quant_kernel<128>, dim3((unsigned)(bh * nblk)), dim3(256), 0, s, p);
        else hipLaunchKernelGGL(sage_quant_kernel<64>, dim3((unsigned)(bh * nblk)), dim3(256), 0, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

}  // extern "C"

// wg_count workgroups starting at workgroup p.wg_base of the problem (0: all of them)
template <int D, int NW>
static int launch_sage_fwd(const SageFwdParams& p, hipStream_t s, int64_t wg_count = 0) {
    using T = SageTile<D>;
    static bool attr_done = false;
    auto kern = sage_fwd_kernel<D, NW>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    constexpr int BM = 32 * NW;
    const int64_t grid = wg_count ? wg_count : (int64_t)((p.Sq + BM - 1) / BM) * p.B * p.H;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * NW), T::LDS_BYTES, s, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

// the first wg_count 256-query workgroups of the problem
template <int D>
static int launch_sage_fwd_wide(const SageFwdParams& p, hipStream_t s, int64_t wg_count) {
    using T = SageWideTile<D>;
    static bool attr_done = false;
    auto kern = sage_fwd_wide_kernel<D>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    if (wg_count > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3((unsigned)wg_count), dim3(256), T::LDS_BYTES, s, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

extern "C" {

int flame_sage_attn_fwd_int8(const void* Qi8, const void* Ki8, const void* q_scales, const void* k_scales,
                             const void* V, void* O, void* LSE, int B, int H, int N_q, int N_kv, int D,
                             float scale, const int64_t* v_strides, const int64_t* o_strides,
                             int64_t v_off, int64_t o_off, int causal, const int32_t* kv_len, void* stream) {
    return flame_sage_attn_fwd_bias_int8(Qi8, Ki8, q_scales, k_scales, V, O, LSE, B, H, N_q, N_kv, D, scale, v_strides,
                                         o_strides, v_off, o_off, causal, kv_len, nullptr, FLAME_ATTN_DTYPE_F32, nullptr,
                                         stream);
}

int flame_sage_attn_fwd_bias_int8(const void* Qi8, const void* Ki8, const void* q_scales, const void* k_scales,
                                  const void* V, void* O, void* LSE, int B, int H, int N_q, int N_kv, int D,
                                  float scale, const int64_t* v_strides, const int64_t* o_strides,
                                  int64_t v_off, int64_t o_off, int causal, const int32_t* kv_len,
                                  const void* bias, int bias_dtype, const int64_t* bias_strides, void* stream) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return FLAME_ATTN_ERR_INVALID;
    if (bias && !bias_strides) return FLAME_ATTN_ERR_INVALID;
    if (bias && bias_dtype != FLAME_ATTN_DTYPE_BF16 && bias_dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;
    if (!(scale > 0.f) || !isfinite(scale)) return FLAME_ATTN_ERR_INVALID;
    if (!Qi8 || !Ki8 || !q_scales || !k_scales) return FLAME_ATTN_ERR_INVALID;
    if (!head_dim_ok(D)) return FLAME_ATTN_ERR_UNSUPPORTED;
    const int Dp = padded_head_dim(D);
    if (!aligned16(Qi8) || !aligned16(Ki8)) return FLAME_ATTN_ERR_UNSUPPORTED;
    int rc;
    if ((rc = check_view(V, v_strides, v_off))) return rc;
    if ((rc = check_view(O, o_strides, o_off))) return rc;
    SageFwdParams p;
    p.d = D;
    p.qi8 = static_cast<const int8_t*>(Qi8);
    p.ki8 = static_cast<const int8_t*>(Ki8);
    p.sq = static_cast<const float*>(q_scales);
    p.sk = static_cast<const float*>(k_scales);
    p.v = static_cast<const uint16_t*>(V) + v_off;
    p.o = static_cast<uint16_t*>(O) + o_off;
    p.lse = static_cast<float*>(LSE);
    p.vs = mk(v_strides); p.os = mk(o_strides);
    p.B = B; p.H = H; p.Sq = N_q; p.Sk = N_kv;
    p.scale = scale;
    p.kv_len = kv_len;
    p.causal = causal ? 1 : 0;
    p.bias = bias;
    if (bias) {
        p.bb = bias_strides[0]; p.bhs = bias_strides[1]; p.bq = bias_strides[2]; p.bk = bias_strides[3];
        p.bias_f32 = bias_dtype == FLAME_ATTN_DTYPE_F32;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    ScopedKernelTimer timer(FLAME_ATTN_KERNEL_SAGE_FWD, s);
    // 256-query workgroups of four 64-query wavefronts (one per SIMD) when they neither add padding rows nor leave
    // compute units without a workgroup, and nothing is excluded; else 128-query workgroups of four 32-query
    // wavefronts.  A last round that would occupy at most half of the compute units with 256-query workgroups is
    // cut into 128-query workgroups in a launch of its own: alone on its compute unit, such a workgroup takes little
    // more than half the time of a 256-query one.
    const int cus = device_cu_count();
    const int64_t n256 = (N_q + 255) / 256, total256 = n256 * B * H;
    const bool wide = n256 * 256 <= ((N_q + 127) / 128) * 128 && total256 >= cus && !causal && !kv_len && !bias &&
                      N_kv % 64 == 0 && wg_waves_override() != 4;
    if (wide) {
        const int64_t rest = total256 % cus;
        const int64_t wide_count = rest <= cus / 2 ? total256 - rest : total256;
        if (2 * total256 > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
        rc = Dp == 128 ? launch_sage_fwd_wide<128>(p, s, wide_count) : launch_sage_fwd_wide<64>(p, s, wide_count);
        if (rc != FLAME_ATTN_OK || wide_count == total256) return rc;
        p.wg_base = (int)(2 * wide_count);
        return Dp == 128 ? launch_sage_fwd<128, 4>(p, s, 2 * rest) : launch_sage_fwd<64, 4>(p, s, 2 * rest);
    }
    if (Dp == 128) return launch_sage_fwd<128, 4>(p, s);
    return launch_sage_fwd<64, 4>(p, s);
}

}  // extern "C"

// the rule for the forward's query tile: 256 rows per workgroup (true) or 128
static bool fwd_rule_wide(int B, int H, int N_q, bool has_mask_or_bias, bool has_kv_len) {
    const int64_t n256 = (N_q + 255) / 256;
    return !has_mask_or_bias && n256 * 256 <= ((int64_t)(N_q + 127) / 128) * 128 && n256 * B * H >= device_cu_count() &&
           !(has_kv_len && n256 * B * H < 2 * device_cu_count()) && wg_waves_override() != 4;
}

static int attn_fwd_impl(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        const void* bias, int bias_dtype, const int64_t* bias_strides,
                        void* stream, int mask_mode = kMaskU8, int Dv = 0, int q_tile_plan = 0, float dropout_p = 0.f,
                        uint64_t dropout_seed = 0, int draw_cq = 0, int draw_ck = 0, FwdScratch scratch = FwdScratch{}) {
    if (Dv == 0) Dv = D;           // V and O may have a head dim of their own (forward only)
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0 || Dv < 0) return FLAME_ATTN_ERR_INVALID;
    if (!(scale > 0.f) || !isfinite(scale)) return FLAME_ATTN_ERR_INVALID;
    // A value head dim above 128 beside a query head dim of at most 128 (the reference's streaming entry point is
    // tested with Dh = 64, Dv = 160: tests/streaming_attn.rs:306-311): the softmax does not depend on V, so O comes
    // out in column ranges of at most 128, each a forward of its own on views of V and O.
    if (head_dim_ok(D) && Dv > 128 && Dv % 8 == 0) {
        for (int c0 = 0; c0 < Dv; c0 += 128) {
            const int rc = attn_fwd_impl(Q, K, V, O, c0 == 0 ? LSE : nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides,
                                         v_strides, o_strides, q_off, k_off, v_off + c0, o_off + c0, lse_off, causal, kv_len,
                                         keep_mask, mask_strides, bias, bias_dtype, bias_strides, stream, mask_mode,
                                         std::min(128, Dv - c0), q_tile_plan, dropout_p, dropout_seed, draw_cq, draw_ck, scratch);
            if (rc != FLAME_ATTN_OK) return rc;
        }
        return FLAME_ATTN_OK;
    }
    // head dims above 128: the forward in chunks of 128, without explicit mask, bias or dropout and with Dv = D
    const bool big = big_head_dim_ok(D) && Dv == D && !keep_mask && !bias && dropout_p == 0.f;
    if (!big && (!head_dim_ok(D) || !head_dim_ok(Dv))) return FLAME_ATTN_ERR_UNSUPPORTED;
    int rc;
    if ((rc = check_view(Q, q_strides, q_off))) return rc;
    if ((rc = check_view(K, k_strides, k_off))) return rc;
    if ((rc = check_view(V, v_strides, v_off))) return rc;
    if ((rc = check_view(O, o_strides, o_off))) return rc;
    if (keep_mask && !mask_strides) return FLAME_ATTN_ERR_INVALID;
    if (bias && !bias_strides) return FLAME_ATTN_ERR_INVALID;
    if (bias && bias_dtype != FLAME_ATTN_DTYPE_BF16 && bias_dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;

    FwdParams p;
    p.q = static_cast<const uint16_t*>(Q) + q_off;
    p.k = static_cast<const uint16_t*>(K) + k_off;
    p.v = static_cast<const uint16_t*>(V) + v_off;
    p.o = static_cast<uint16_t*>(O) + o_off;
    p.lse = LSE ? static_cast<float*>(LSE) + lse_off : nullptr;
    p.qs = mk(q_strides); p.ks = mk(k_strides); p.vs = mk(v_strides); p.os = mk(o_strides);
    p.B = B; p.H = H; p.Sq = N_q; p.Sk = N_kv;
    p.d = D;
    p.dv = Dv;
    p.scale = scale;
    p.m.kv_len = kv_len;
    p.m.mask = keep_mask;
    p.m.sb = keep_mask ? mask_strides[0] : 0;
    p.m.sh = keep_mask ? mask_strides[1] : 0;
    p.m.sq = keep_mask ? mask_strides[2] : 0;
    p.m.sk = keep_mask ? mask_strides[3] : 0;
    p.m.mask_mode = mask_mode;
    p.m.rows16 = keep_mask && mask_mode == kMaskU8 && p.m.sk == 1 &&
                 (reinterpret_cast<uintptr_t>(keep_mask) | (uintptr_t)p.m.sb | (uintptr_t)p.m.sh | (uintptr_t)p.m.sq) % 16 == 0;
    p.m.causal = causal ? 1 : 0;
    p.m.bias = bias;
    if (bias) {
        p.m.bb = bias_strides[0]; p.m.bh = bias_strides[1]; p.m.bq = bias_strides[2]; p.m.bk = bias_strides[3];
        p.m.bias_f32 = bias_dtype == FLAME_ATTN_DTYPE_F32;
        p.m.inv_scale = 1.0f / scale;
    }

    hipStream_t s = static_cast<hipStream_t>(stream);
    if (big) return D <= 256 ? launch_fwd_bigd<2>(p, s, scratch) : D <= 384 ? launch_fwd_bigd<3>(p, s, scratch) : launch_fwd_bigd<4>(p, s, scratch);
    const bool hm = keep_mask != nullptr || bias != nullptr;
    if (dropout_p != 0.f) {
        if (!set_dropout(p.m, dropout_p, dropout_seed, draw_cq, draw_ck, N_q, N_kv)) return FLAME_ATTN_ERR_INVALID;
        if (std::max(padded_head_dim(D), padded_head_dim(Dv)) == 128)
            return hm ? launch_fwd_dropout<128, true>(p, s) : launch_fwd_dropout<128, false>(p, s);
        return hm ? launch_fwd_dropout<64, true>(p, s) : launch_fwd_dropout<64, false>(p, s);
    }
    // 256-query workgroups when they neither add padding rows nor leave compute units
    // without a workgroup
    bool wide = fwd_rule_wide(B, H, N_q, hm, kv_len != nullptr);
    // a plan (128 or 256 query rows per workgroup) overrides the rule where the kernels leave the choice open
    if (q_tile_plan == 128) wide = false;
    else if (q_tile_plan == 256 && !hm) wide = true;
    // ... as 4 wavefronts of 64 queries when nothing is excluded at all, else as 8 wavefronts of 32
    const bool plain = !causal && kv_len == nullptr && N_kv % 64 == 0;
    // a keep-mask with vector-loadable rows over whole tiles and no bias: the lean masked kernel
    const int DP = std::max(padded_head_dim(D), padded_head_dim(Dv));
    if (keep_mask != nullptr && bias == nullptr && p.m.rows16 && N_kv % 64 == 0)
        return DP == 128 ? launch_fwd<128, true, 4, true>(p, s) : launch_fwd<64, true, 4, true>(p, s);
    if (DP == 128)
        return hm ? launch_fwd<128, true, 4>(p, s)
                  : wide ? (plain ? launch_fwd_wide<128>(p, s) : launch_fwd<128, false, 8>(p, s)) : launch_fwd<128, false, 4>(p, s);
    return hm ? launch_fwd<64, true, 4>(p, s)
              : wide ? (plain ? launch_fwd_wide<64>(p, s) : launch_fwd<64, false, 8>(p, s)) : launch_fwd<64, false, 4>(p, s);
}


extern "C" {

int flame_attn_fwd_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* stream) {
    return attn_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_off, k_off, v_off, o_off, lse_off, causal, kv_len, keep_mask, mask_strides,
                         nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream);
}

size_t flame_attn_fwd_workspace_bytes(int B, int H, int N_q, int N_kv, int D) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || !big_head_dim_ok(D)) return 0;
    const int bm = bigd_query_tile(D);
    const int ks = bigd_key_splits((int64_t)((N_q + bm - 1) / bm) * B * H, N_kv);
    return ks > 1 ? bigd_partials_bytes(ks, (int64_t)B * H * N_q, D) : 0;
}

int flame_attn_fwd_ws_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                           int B, int H, int N_q, int N_kv, int D, float scale,
                           const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                           const int64_t* o_strides,
                           int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                           int causal, const int32_t* kv_len,
                           const uint8_t* keep_mask, const int64_t* mask_strides,
                           void* workspace, size_t workspace_bytes, void* stream) {
    if (workspace && !aligned16(workspace)) return FLAME_ATTN_ERR_UNSUPPORTED;
    FwdScratch sc;
    sc.ws = workspace;
    sc.bytes = workspace ? workspace_bytes : 0;
    return attn_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_off, k_off, v_off, o_off, lse_off, causal, kv_len, keep_mask, mask_strides,
                         nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, 0, 0, 0.f, 0, 0, 0, sc);
}

int flame_attn_fwd_dropout_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                float dropout_p, uint64_t dropout_seed, void* stream) {
    return attn_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_off, k_off, v_off, o_off, lse_off, causal, kv_len, keep_mask, mask_strides,
                         nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, 0, 0, dropout_p, dropout_seed);
}

int flame_attn_fwd_dropout_tiled_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                      int B, int H, int N_q, int N_kv, int D, float scale,
                                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                      const int64_t* o_strides,
                                      int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                      int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                      float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv, void* stream) {
    return attn_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_off, k_off, v_off, o_off, lse_off, causal, kv_len, keep_mask, mask_strides,
                         nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, 0, 0, dropout_p, dropout_seed, draw_chunk_q,
                         draw_chunk_kv);
}

int flame_attn_fwd_bias_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                             int B, int H, int N_q, int N_kv, int D, float scale,
                             const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                             const int64_t* o_strides,
                             int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                             const void* bias, int bias_dtype, const int64_t* bias_strides,
                             const uint8_t* keep_mask, const int64_t* mask_strides,
                             void* stream) {
    if (!bias) return FLAME_ATTN_ERR_INVALID;
    return attn_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_off, k_off, v_off, o_off, lse_off, 0, nullptr, keep_mask, mask_strides,
                         bias, bias_dtype, bias_strides, stream);
}

// ------------------------------------------------------------------------------------------------
// Entry points with the names and argument lists of the reference's FFI for this path.  They are
// thin shims onto the forward and backward above.  Their argument lists have no workspace, and the
// reference's own implementations allocate behind them (a workspace per cached graph,
// src/cuda/cudnn_sdpa.cpp:204-212; eleven buffers per call, cuda/sdpa_stream_bf16.cu:214-239): where a
// kernel needs scratch they take the library's per-(device, stream) buffer.
// ------------------------------------------------------------------------------------------------
static int mat_fwd_impl(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                        const void* bias, int bias_dtype, const int64_t* bias_strides,
                        void* workspace, size_t workspace_bytes, void* stream, int mask_mode,
                        float dropout_p = 0.f, uint64_t dropout_seed = 0, int draw_cq = 0, int draw_ck = 0);
static FwdScratch library_scratch() {
    FwdScratch sc;
    sc.library = true;
    return sc;
}

int flame_cudnn_sdpa_bf16(const void* Q, const void* K, const void* V, void* O,
                          int B, int H, int N_q, int N_kv, int D, float scale,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides,
                          int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                          int64_t o_offset_elems, void* stream) {
    return attn_fwd_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_offset_elems, k_offset_elems, v_offset_elems, o_offset_elems, 0, 0, nullptr, nullptr, nullptr,
                         nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, 0, 0, 0.f, 0, 0, 0, library_scratch());
}

int flame_cudnn_sdpa_bf16_train_fwd(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                    int B, int H, int N_q, int N_kv, int D, float scale,
                                    const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                    const int64_t* o_strides,
                                    int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                                    int64_t o_offset_elems, int64_t stats_offset_elems, void* stream) {
    if (!Stats) return FLAME_ATTN_ERR_INVALID;
    return attn_fwd_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides, o_strides,
                         q_offset_elems, k_offset_elems, v_offset_elems, o_offset_elems, stats_offset_elems, 0, nullptr,
                         nullptr, nullptr, nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, 0, 0, 0.f, 0, 0, 0,
                         library_scratch());
}

}  // extern "C"

namespace {
// Scratch for the reference-named entry points, whose argument lists have no workspace: one lazily grown
// buffer per (device, stream), as the reference's shim keeps a workspace it allocated once per shape.
// Calls on one stream are ordered, so they may share a buffer; calls on different streams get
// different buffers and cannot race; host threads that share a stream are kept apart by
// g_lib_scratch_enqueue_mu, which an entry point holds from taking the buffer to its last launch (otherwise
// the kernels of two calls could interleave on the stream and read each other's rows).
// hipMalloc happens on first use or growth only; under a stream capture a call that would have to allocate
// returns FLAME_ATTN_ERR_UNSUPPORTED instead (an allocation there would invalidate the capture).  An outgrown
// buffer is freed at once when its stream is idle, else at a later call that finds the stream idle: a
// kernel still running on it keeps valid memory.
struct BwdScratchSlot {
    int dev;
    hipStream_t stream;
    void* ptr;
    size_t bytes;
};
struct BwdScratch {
    std::mutex mu;
    std::vector<BwdScratchSlot> slots;
    std::vector<BwdScratchSlot> retired;      // outgrown buffers whose stream was busy when they were replaced
};
BwdScratch g_bwd_scratch;
std::mutex g_lib_scratch_enqueue_mu;

bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

int bwd_scratch_get(size_t need, hipStream_t stream, void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    std::lock_guard<std::mutex> g(g_bwd_scratch.mu);
    BwdScratchSlot* slot = nullptr;
    for (auto& sl : g_bwd_scratch.slots)
        if (sl.dev == dev && sl.stream == stream) slot = &sl;
    if (!slot) {
        g_bwd_scratch.slots.push_back(BwdScratchSlot{dev, stream, nullptr, 0});
        slot = &g_bwd_scratch.slots.back();
    }
    const bool capturing = stream_is_capturing(stream);
    auto idle = [&]() {
        if (capturing) return false;
        if (hipStreamQuery(stream) == hipSuccess) return true;
        (void)hipGetLastError();       // hipErrorNotReady
        return false;
    };
    if (!g_bwd_scratch.retired.empty()) {
        bool is_idle = false, asked = false;
        for (size_t i = 0; i < g_bwd_scratch.retired.size();) {
            BwdScratchSlot& r = g_bwd_scratch.retired[i];
            if (r.dev == dev && r.stream == stream) {
                if (!asked) { is_idle = idle(); asked = true; }
                if (is_idle) {
                    (void)hipFree(r.ptr);
                    g_bwd_scratch.retired.erase(g_bwd_scratch.retired.begin() + (long)i);
                    continue;
                }
            }
            ++i;
        }
    }
    if (slot->bytes < need) {
        if (capturing) return FLAME_ATTN_ERR_UNSUPPORTED;
        void* fresh = nullptr;
        e = hipMalloc(&fresh, need);
        if (e != hipSuccess) return (int)e;
        if (slot->ptr) {
            if (idle()) (void)hipFree(slot->ptr);
            else g_bwd_scratch.retired.push_back(BwdScratchSlot{dev, stream, slot->ptr, slot->bytes});
        }
        slot->ptr = fresh;
        slot->bytes = need;
    }
    *out = slot->ptr;
    return FLAME_ATTN_OK;
}
// The key-split forward for head dims above 128 takes its partial outputs from the same buffers: work on one stream
// is ordered, so a forward's partials are merged before a later backward on that stream writes there.
int lib_scratch_get(size_t need, hipStream_t stream, void** out) { return bwd_scratch_get(need, stream, out); }
std::mutex& lib_scratch_enqueue_mutex() { return g_lib_scratch_enqueue_mu; }

// Scratch of the allocation-free backward: a fixed array in device memory that every GPU the library
// runs on holds until the process ends.  Layout as the caller workspace of flame_attn_bwd_bf16: two fp32
// rows per query (at most FLAME_ATTN_NOALLOC_MAX_ROWS queries over all batches and heads), then the fp32
// dK/dV partial sums of the split key blocks.  The name below is a host-side stand-in: the address the
// kernels are given comes from hipGetSymbolAddress, once per device.
constexpr size_t kNoallocRowsBytes = 2 * (size_t)FLAME_ATTN_NOALLOC_MAX_ROWS * sizeof(float);
constexpr size_t kNoallocSplitBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kNoallocRowsBytes + kNoallocSplitBytes];

struct NoallocScratch {
    std::mutex mu;
    void* ptr[64] = {};
};
NoallocScratch g_noalloc;

int noalloc_scratch_get(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return FLAME_ATTN_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> g(g_noalloc.mu);
    if (!g_noalloc.ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return FLAME_ATTN_ERR_UNSUPPORTED;
        g_noalloc.ptr[dev] = ptr;
    }
    *out = g_noalloc.ptr[dev];
    return FLAME_ATTN_OK;
}

// bf16 keep-mask (>= 0.5 attends) -> uint8 keep-mask, contiguous
__global__ void mask_bf16_to_u8_kernel(const uint16_t* src, uint8_t* dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = __builtin_bit_cast(float, (uint32_t)src[i] << 16) >= 0.5f ? 1 : 0;
}
__global__ void mask_f32_to_u8_kernel(const float* src, uint8_t* dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i] >= 0.5f ? 1 : 0;
}
__global__ void cast_f32_to_bf16_kernel(const float* src, uint16_t* dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = (uint16_t)(pack_bf16(src[i], 0.f) & 0xffffu);
}
// gradient accumulation of the host layer: acc += float(g) with g bf16 or fp32; fill with a constant
__global__ void accumulate_f32_kernel(float* acc, const void* g, int g_is_f32, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = g_is_f32 ? static_cast<const float*>(g)[i]
                                 : __uint_as_float((uint32_t)static_cast<const uint16_t*>(g)[i] << 16);
        acc[i] += v;
    }
}
__global__ void fill_kernel(void* dst, float value, int is_f32, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        if (is_f32) static_cast<float*>(dst)[i] = value;
        else static_cast<uint16_t*>(dst)[i] = (uint16_t)(pack_bf16(value, 0.f) & 0xffffu);
    }
}
}  // namespace

extern "C" {

int flame_cudnn_sdpa_bwd_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                              const void* Stats, void* dQ, void* dK, void* dV,
                              int B, int H, int N_q, int N_kv, int D, float scale,
                              const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                              const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                              const int64_t* dk_strides, const int64_t* dv_strides,
                              int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                              int64_t o_offset_elems, int64_t do_offset_elems, int64_t stats_offset_elems,
                              int64_t dq_offset_elems, int64_t dk_offset_elems, int64_t dv_offset_elems,
                              void* stream) {
    const size_t need = flame_attn_bwd_workspace_bytes(B, H, N_q, D);
    if (need == 0) return FLAME_ATTN_ERR_INVALID;
    std::lock_guard<std::mutex> enqueue(g_lib_scratch_enqueue_mu);      // from taking the buffer to the last launch
    void* ws = nullptr;
    int rc = bwd_scratch_get(need, static_cast<hipStream_t>(stream), &ws);
    if (rc) return rc;
    return flame_attn_bwd_bf16(Q, K, V, O, dO, Stats, dQ, dK, dV, B, H, N_q, N_kv, D, scale, q_strides, k_strides,
                               v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides, q_offset_elems,
                               k_offset_elems, v_offset_elems, o_offset_elems, do_offset_elems, stats_offset_elems,
                               dq_offset_elems, dk_offset_elems, dv_offset_elems, 0, nullptr, nullptr, nullptr, ws,
                               need, stream);
}

int flame_attn_bwd_noalloc_max_rows(void) { return FLAME_ATTN_NOALLOC_MAX_ROWS; }

int flame_attn_bwd_bf16_noalloc(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                const void* LSE, void* dQ, void* dK, void* dV,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                const int64_t* dk_strides, const int64_t* dv_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                int causal, const int32_t* kv_len,
                                const uint8_t* keep_mask, const int64_t* mask_strides, void* stream) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return FLAME_ATTN_ERR_INVALID;
    if ((int64_t)B * H * N_q > FLAME_ATTN_NOALLOC_MAX_ROWS) return FLAME_ATTN_ERR_TOO_LARGE;
    void* ws = nullptr;
    int rc = noalloc_scratch_get(&ws);
    if (rc) return rc;
    // The row part is sized for this call, so the partial sums start where flame_attn_bwd_bf16 expects
    // them; every byte the kernels read from the scratch was written earlier in the same call.
    const size_t bytes = bwd_rows_bytes(B, H, N_q) + kNoallocSplitBytes;
    return flame_attn_bwd_bf16(Q, K, V, O, dO, LSE, dQ, dK, dV, B, H, N_q, N_kv, D, scale, q_strides, k_strides,
                               v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides, q_off, k_off,
                               v_off, o_off, do_off, lse_off, dq_off, dk_off, dv_off, causal, kv_len, keep_mask,
                               mask_strides, ws, bytes, stream);
}

int flame_flash_attention_bf16(const void* Q, const void* K, const void* V, void* O, float* LSE,
                               int batch_heads, int seq_len_q, int seq_len_kv, int head_dim, void* stream) {
    if (batch_heads <= 0 || seq_len_q <= 0 || seq_len_kv <= 0 || head_dim <= 0) return FLAME_ATTN_ERR_INVALID;
    const int64_t qs[4] = {(int64_t)seq_len_q * head_dim, (int64_t)seq_len_q * head_dim, head_dim, 1};
    const int64_t ks[4] = {(int64_t)seq_len_kv * head_dim, (int64_t)seq_len_kv * head_dim, head_dim, 1};
    return attn_fwd_impl(Q, K, V, O, LSE, batch_heads, 1, seq_len_q, seq_len_kv, head_dim, 1.0f / sqrtf((float)head_dim),
                         qs, ks, ks, qs, 0, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr, nullptr, FLAME_ATTN_DTYPE_F32, nullptr,
                         stream, kMaskU8, 0, 0, 0.f, 0, 0, 0, library_scratch());
}

static FlameAttnStatus to_status(int rc) {
    if (rc == FLAME_ATTN_OK) return FLAME_ATTN_STATUS_OK;
    if (rc == FLAME_ATTN_ERR_INVALID) return FLAME_ATTN_STATUS_ERR_INVALID;
    if (rc == FLAME_ATTN_ERR_UNSUPPORTED) return FLAME_ATTN_STATUS_ERR_UNSUPPORTED;
    return FLAME_ATTN_STATUS_ERR_HIP;
}

FlameAttnStatus flame_sdpa_chunked_bf16(const void* q, const void* k, const void* v, int B, int H, int Q, int K,
                                        int Dh, int Dv, float scale, int chunk, int causal, int mask_heads,
                                        const void* mask, void* out, void* workspace, uint64_t workspace_bytes,
                                        void* stream) {
    if (!q || !k || !v || !out) return FLAME_ATTN_STATUS_ERR_INVALID;
    if (B <= 0 || H <= 0 || Q < 0 || K < 0 || Dh <= 0 || Dv <= 0) return FLAME_ATTN_STATUS_ERR_INVALID;
    if (Q == 0 || K == 0) return FLAME_ATTN_STATUS_OK;
    if (chunk <= 0) return FLAME_ATTN_STATUS_ERR_INVALID;
    const int64_t qs[4] = {(int64_t)H * Q * Dh, (int64_t)Q * Dh, Dh, 1};
    const int64_t ks[4] = {(int64_t)H * K * Dh, (int64_t)K * Dh, Dh, 1};
    const int64_t vs[4] = {(int64_t)H * K * Dv, (int64_t)K * Dv, Dv, 1};     // V [B,H,K,Dv], out [B,H,Q,Dv]
    const int64_t os[4] = {(int64_t)H * Q * Dv, (int64_t)Q * Dv, Dv, 1};
    // bf16 keep-mask [B, mask_heads, Q, K], a value below 0.5 excludes: read in place by the masked kernel, so
    // the workspace (which the reference sizes for its own score chunks) is not needed at all
    (void)workspace; (void)workspace_bytes;
    int64_t ms[4] = {0, 0, 0, 0};
    if (mask) {
        if (mask_heads != 1 && mask_heads != H) return FLAME_ATTN_STATUS_ERR_INVALID;
        ms[0] = (int64_t)mask_heads * Q * K;
        ms[1] = mask_heads == 1 ? 0 : (int64_t)Q * K;
        ms[2] = K;
        ms[3] = 1;
    }
    auto run = [&](int q_tile) {
        const int rc = attn_fwd_impl(q, k, v, out, nullptr, B, H, Q, K, Dh, scale, qs, ks, vs, os, 0, 0, 0, 0, 0, causal, nullptr,
                                     static_cast<const uint8_t*>(mask), mask ? ms : nullptr, nullptr, FLAME_ATTN_DTYPE_F32, nullptr,
                                     stream, kMaskBf16Keep, Dv, q_tile, 0.f, 0, 0, 0, library_scratch());
        if (rc != FLAME_ATTN_ERR_UNSUPPORTED) return rc;
        // The reference's entry point takes any head dims (its scalar kernels, cuda/src/flame_sdpa_stub.cu:696-866):
        // what the fused kernels do not serve goes through materialised scores, in the library's own scratch.
        const size_t need = flame_attn_materialised_workspace_bytes(B, H, Q, K, Dh, Dv, 0);
        std::lock_guard<std::mutex> enqueue(lib_scratch_enqueue_mutex());
        void* ws = nullptr;
        const int rs = lib_scratch_get(need, static_cast<hipStream_t>(stream), &ws);
        if (rs) return rs;
        return mat_fwd_impl(q, k, v, out, nullptr, B, H, Q, K, Dh, Dv, scale, qs, ks, vs, os, 0, 0, 0, 0, 0, causal, nullptr,
                            static_cast<const uint8_t*>(mask), mask ? ms : nullptr, nullptr, FLAME_ATTN_DTYPE_F32, nullptr, ws, need,
                            stream, kMaskBf16Keep);
    };
    // ---- the launch plan: the query tile of a workgroup (see plan_cache.hpp)
    PlanCache& pc = PlanCache::instance();
    const PlanConfig& cfg = pc.config();
    // the masked kernels come with 128-row workgroups only, and head dims other than the multiples of 8 up to 128 have
    // one kernel (or the materialised path): nothing to choose, so nothing is measured
    const bool one_tile = mask != nullptr || !head_dim_ok(Dh);
    const int rule_q = (!one_tile && fwd_rule_wide(B, H, Q, false, false)) ? 256 : 128;
    const PlanKey key{B, H, Q, K, Dh, Dv, mask ? mask_heads : 0, causal ? 1 : 0};
    int q_tile = rule_q;
    uint64_t source = kPlanRule, candidates = 1, best_ns = 0;
    if (cfg.q_override > 0) {
        q_tile = (cfg.q_override <= 128 || one_tile) ? 128 : 256;
        source = kPlanForced;
        pc.with_stats([&](FlameSdpaAutotuneStats& st) {
            st.env_forced += 1;
            if (q_tile != cfg.q_override) st.clamped += 1;
        });
    } else if (cfg.enabled) {
        Plan plan;
        const bool hit = pc.lookup(key, &plan) && (plan.q_tile == 128 || (plan.q_tile == 256 && !one_tile)) && plan.k_tile == 64;
        pc.with_stats([&](FlameSdpaAutotuneStats& st) { (hit ? st.cache_hits : st.cache_misses) += 1; });
        if (hit) {
            q_tile = plan.q_tile;
            source = kPlanCacheHit;
        } else {
            hipStream_t hs = static_cast<hipStream_t>(stream);
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(hs, &capturing) != hipSuccess) (void)hipGetLastError();
            if (one_tile || capturing != hipStreamCaptureStatusNone) {
                pc.with_stats([&](FlameSdpaAutotuneStats& st) { st.skipped += 1; });
            } else {
                // both tiles on the caller's own problem: the forward only reads its inputs, so running it several
                // times leaves the same output
                double ms_of[2] = {0, 0};
                bool ok = true;
                hipEvent_t e0 = nullptr, e1 = nullptr;
                ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
                for (int c = 0; c < 2 && ok; ++c) {
                    const int cand = c == 0 ? 128 : 256;
                    for (int i = 0; i < cfg.warmups && ok; ++i) ok = run(cand) == FLAME_ATTN_OK;
                    ok = ok && hipEventRecord(e0, hs) == hipSuccess;
                    for (int i = 0; i < cfg.repeats && ok; ++i) ok = run(cand) == FLAME_ATTN_OK;
                    float ms_f = 0.f;
                    ok = ok && hipEventRecord(e1, hs) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
                         hipEventElapsedTime(&ms_f, e0, e1) == hipSuccess;
                    ms_of[c] = ms_f / cfg.repeats;
                }
                if (e0) (void)hipEventDestroy(e0);
                if (e1) (void)hipEventDestroy(e1);
                if (ok) {
                    // within the tie margin the rule's tile stays
                    const int fastest = ms_of[0] <= ms_of[1] ? 128 : 256;
                    const double t_fast = std::min(ms_of[0], ms_of[1]), t_rule = ms_of[rule_q == 128 ? 0 : 1];
                    q_tile = (t_rule <= t_fast * (1.0 + cfg.tie_eps)) ? rule_q : fastest;
                    source = kPlanTuned;
                    candidates = 2;
                    best_ns = (uint64_t)(ms_of[q_tile == 128 ? 0 : 1] * 1e6);
                    pc.with_stats([&](FlameSdpaAutotuneStats& st) { st.tuned += 1; });
                } else {
                    (void)hipGetLastError();
                    pc.with_stats([&](FlameSdpaAutotuneStats& st) {
                        st.errors += 1;
                        st.fallback += 1;
                    });
                }
            }
            pc.store(key, q_tile, 64);
        }
    }
    const int rc = run(q_tile);
    pc.with_stats([&](FlameSdpaAutotuneStats& st) {
        if (rc != FLAME_ATTN_OK) {
            st.errors += 1;
            return;
        }
        st.last_q_chunk = (uint64_t)q_tile;
        st.last_k_chunk = 64;
        st.last_candidate_count = candidates;
        st.last_best_time_ns = best_ns;
        st.last_plan_source = source;
        st.last_shape_b = (uint64_t)B; st.last_shape_h = (uint64_t)H; st.last_shape_q = (uint64_t)Q; st.last_shape_k = (uint64_t)K;
        st.last_shape_dh = (uint64_t)Dh; st.last_shape_dv = (uint64_t)Dv;
        st.last_shape_mask_heads = (uint64_t)(mask ? mask_heads : 0);
        st.last_shape_causal = causal ? 1 : 0;
    });
    return to_status(rc);
}

int flame_sdpa_autotune_get_stats(FlameSdpaAutotuneStats* out) {
    if (!out) return FLAME_ATTN_STATUS_ERR_INVALID;     // 1, as cuda/src/flame_sdpa_stub.cu:1382-1385
    PlanCache::instance().get_stats(out);
    return FLAME_ATTN_OK;
}

int flame_sdpa_autotune_reset_stats(void) {
    PlanCache::instance().reset_stats();
    return FLAME_ATTN_OK;
}

int flame_sdpa_autotune_flush_cache(void) {
    PlanCache::instance().flush();
    return FLAME_ATTN_OK;
}

int streaming_attn_bf16_fp32_launch(const void* Q, const void* K, const void* V, int B, int H, int S, int Dh, int Dv,
                                    long qB, long qH, long qS, long qD, long kB, long kH, long kS, long kD,
                                    long vB, long vH, long vS, long vD, void* O, long oB, long oH, long oS, long oD,
                                    float scale, int chunk_size, int causal, const uint8_t* k_pad_mask,
                                    void* stream) {
    if (chunk_size <= 0) return FLAME_ATTN_ERR_INVALID;
    const int64_t qs[4] = {qB, qH, qS, qD}, ks[4] = {kB, kH, kS, kD}, vs[4] = {vB, vH, vS, vD}, os[4] = {oB, oH, oS, oD};
    const int64_t ms[4] = {(int64_t)H * S, S, 0, 1};     // [B,H,S] key-padding mask, 0 = excluded
    return attn_fwd_impl(Q, K, V, O, nullptr, B, H, S, S, Dh, scale, qs, ks, vs, os, 0, 0, 0, 0, 0, causal, nullptr,
                         k_pad_mask, k_pad_mask ? ms : nullptr, nullptr, FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskU8, Dv, 0, 0.f,
                         0, 0, 0, library_scratch());
}

bool sdpa_stream_bf16_launch(const void* dQ, const void* dK, const void* dV, void* dO, int B, int H, int Q_len,
                             int K_len, int d, float scale, const void* attn_mask, int64_t mask_stride_ek,
                             int64_t mask_stride_eq, int64_t mask_stride_eh, int64_t mask_stride_eb, int head_tile,
                             int q_tile, int max_q_tile, void* stream, char* unsupported_reason, int reason_buflen) {
    auto fail = [&](const char* why) {
        if (unsupported_reason && reason_buflen > 0) snprintf(unsupported_reason, (size_t)reason_buflen, "%s", why);
        return false;
    };
    (void)head_tile;
    if (q_tile > max_q_tile) return fail("q_tile exceeds max_q_tile");
    if (!head_dim_ok(d) && !(big_head_dim_ok(d) && !attn_mask))
        return fail("head dim must be a multiple of 8, at most 128 (at most 512 without a mask)");
    const int64_t qs[4] = {(int64_t)H * Q_len * d, (int64_t)Q_len * d, d, 1};
    const int64_t ks[4] = {(int64_t)H * K_len * d, (int64_t)K_len * d, d, 1};
    // bf16 mask addressed by the caller's four element strides; in this entry point a value above 0.5 EXCLUDES
    const int64_t ms[4] = {mask_stride_eb, mask_stride_eh, mask_stride_eq, mask_stride_ek};
    const int rc = attn_fwd_impl(dQ, dK, dV, dO, nullptr, B, H, Q_len, K_len, d, scale, qs, ks, ks, qs, 0, 0, 0, 0, 0, 0,
                                 nullptr, static_cast<const uint8_t*>(attn_mask), attn_mask ? ms : nullptr, nullptr,
                                 FLAME_ATTN_DTYPE_F32, nullptr, stream, kMaskBf16Drop, 0, 0, 0.f, 0, 0, 0, library_scratch());
    if (rc != FLAME_ATTN_OK) return fail(rc == FLAME_ATTN_ERR_INVALID ? "invalid argument" : "unsupported shape or HIP error");
    if (unsupported_reason && reason_buflen > 0) unsupported_reason[0] = 0;
    return true;
}

int flame_attn_convert_keep_mask(const void* src, int src_dtype, void* dst_u8, int64_t n, void* stream) {
    if (!src || !dst_u8 || n <= 0) return FLAME_ATTN_ERR_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (n > (int64_t)0x7fffffff * 256) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (src_dtype == FLAME_ATTN_DTYPE_BF16)
        hipLaunchKernelGGL(mask_bf16_to_u8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(src),
                           static_cast<uint8_t*>(dst_u8), n);
    else if (src_dtype == FLAME_ATTN_DTYPE_F32)
        hipLaunchKernelGGL(mask_f32_to_u8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const float*>(src),
                           static_cast<uint8_t*>(dst_u8), n);
    else
        return FLAME_ATTN_ERR_UNSUPPORTED;
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int flame_attn_cast_f32_to_bf16(const void* src_f32, void* dst_bf16, int64_t n, void* stream) {
    if (!src_f32 || !dst_bf16 || n <= 0) return FLAME_ATTN_ERR_INVALID;
    if (n > (int64_t)0x7fffffff * 256) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(cast_f32_to_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const float*>(src_f32),
                       static_cast<uint16_t*>(dst_bf16), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int flame_attn_accumulate_f32(void* acc_f32, const void* grad, int grad_dtype, int64_t n, void* stream) {
    if (!acc_f32 || !grad || n <= 0) return FLAME_ATTN_ERR_INVALID;
    if (grad_dtype != FLAME_ATTN_DTYPE_BF16 && grad_dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;
    if (n > (int64_t)0x7fffffff * 256) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(accumulate_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<float*>(acc_f32), grad,
                       grad_dtype == FLAME_ATTN_DTYPE_F32 ? 1 : 0, n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int flame_attn_fill(void* dst, int dtype, float value, int64_t n, void* stream) {
    if (!dst || n <= 0) return FLAME_ATTN_ERR_INVALID;
    if (dtype != FLAME_ATTN_DTYPE_BF16 && dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;
    if (n > (int64_t)0x7fffffff * 256) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       dst, value, dtype == FLAME_ATTN_DTYPE_F32 ? 1 : 0, n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int flame_attn_prep_rmsnorm_rope_bf16(const void* X, const void* weight, const void* cos, const void* sin,
                                      int table_dtype, void* Y, int B, int H, int N, int D, float eps,
                                      int apply_norm, const int64_t* x_strides, const int64_t* y_strides,
                                      int64_t x_off, int64_t y_off, void* stream) {
    if (!X || !Y || !x_strides || !y_strides || B <= 0 || H <= 0 || N <= 0) return FLAME_ATTN_ERR_INVALID;
    if ((cos == nullptr) != (sin == nullptr)) return FLAME_ATTN_ERR_INVALID;
    if (D != 64 && D != 128) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (table_dtype != FLAME_ATTN_DTYPE_BF16 && table_dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;
    if (int rc = check_view(X, x_strides, x_off)) return rc;
    if (int rc = check_view(Y, y_strides, y_off)) return rc;
    if (weight && !aligned16(weight)) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (cos && (!aligned16(cos) || !aligned16(sin))) return FLAME_ATTN_ERR_UNSUPPORTED;
    PrepParams p{};
    p.x = static_cast<const uint16_t*>(X) + x_off;
    p.y = static_cast<uint16_t*>(Y) + y_off;
    p.w = static_cast<const uint16_t*>(weight);
    p.cos_t = cos;
    p.sin_t = sin;
    p.xs = mk(x_strides);
    p.ys = mk(y_strides);
    p.B = B;
    p.H = H;
    p.N = N;
    p.eps = eps;
    p.norm = apply_norm ? 1 : 0;
    p.table_f32 = table_dtype == FLAME_ATTN_DTYPE_F32;
    const int64_t items = (int64_t)B * N * ((H + kPrepHeadsPerThread - 1) / kPrepHeadsPerThread);   // (position, head group)
    const int rpb = 256 / (D / 8);
    const int64_t grid = (items + rpb - 1) / rpb;
    if (grid > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    {
        ScopedKernelTimer t(FLAME_ATTN_KERNEL_INPUT_PREP, s);
        if (D == 128) hipLaunchKernelGGL(prep_qk_kernel<128>, dim3((unsigned)grid), dim3(256), 0, s, p);
        else hipLaunchKernelGGL(prep_qk_kernel<64>, dim3((unsigned)grid), dim3(256), 0, s, p);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

// ---- element-wise primitives on score tiles, under the reference's names; 0 = launched, 1 = not (the
// reference's convention for these symbols: src/kernels/sdpa_kernels.cu:232-403)

static int tile_launched() { return hipGetLastError() == hipSuccess ? 0 : 1; }
static bool tile_grid(int64_t n_threads, unsigned* grid) {
    const int64_t g = (n_threads + 255) / 256;
    if (g > 0x7fffffff) return false;
    *grid = (unsigned)g;
    return true;
}

int flame_apply_causal_mask_fp32(float* scores, int B, int H, int Q, int K, int q_offset, int k_offset, void* stream) {
    if (B < 0 || H < 0 || Q < 0 || K < 0) return 1;
    const int64_t total = (int64_t)B * H * Q * K;
    if (total == 0) return 0;
    if (!scores) return 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned grid;
    if (K % 4 == 0 && aligned16(scores)) {
        if (!tile_grid(total / 4, &grid)) return 1;
        hipLaunchKernelGGL(tile_causal_mask_kernel<4>, dim3(grid), dim3(256), 0, s, scores, total / 4, Q, K, q_offset, k_offset);
    } else {
        if (!tile_grid(total, &grid)) return 1;
        hipLaunchKernelGGL(tile_causal_mask_kernel<1>, dim3(grid), dim3(256), 0, s, scores, total, Q, K, q_offset, k_offset);
    }
    return tile_launched();
}

int flame_apply_attn_mask_fp32(float* scores, const uint8_t* mask, int B, int H, int Q, int K, void* stream) {
    if (B < 0 || H < 0 || Q < 0 || K < 0) return 1;
    const int64_t total = (int64_t)B * H * Q * K;
    if (total == 0) return 0;
    if (!scores || !mask) return 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned grid;
    if (total % 4 == 0 && aligned16(scores) && (reinterpret_cast<uintptr_t>(mask) & 3) == 0) {
        if (!tile_grid(total / 4, &grid)) return 1;
        hipLaunchKernelGGL(tile_attn_mask_kernel<4>, dim3(grid), dim3(256), 0, s, scores, mask, total / 4);
    } else {
        if (!tile_grid(total, &grid)) return 1;
        hipLaunchKernelGGL(tile_attn_mask_kernel<1>, dim3(grid), dim3(256), 0, s, scores, mask, total);
    }
    return tile_launched();
}

int flame_sdpa_add_mask_tile_fp32(float* logits, const uint8_t* user_bool, const float* user_add, int BH, int q_t, int k_t,
                                  int q_abs_start, int k_abs_start, int user_bool_rank, int user_add_rank, int k_total,
                                  int bool_zero_is_mask, int causal_flag, void* stream) {
    if (BH < 0 || q_t < 0 || k_t < 0) return 1;
    const int64_t total = (int64_t)BH * q_t * k_t;
    if (total == 0) return 0;
    if (!logits) return 1;
    TileMaskParams p{logits, user_bool, user_add, q_t, k_t, q_abs_start, k_abs_start, user_bool_rank, user_add_rank, k_total,
                     bool_zero_is_mask != 0, causal_flag != 0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned grid;
    if (k_t % 4 == 0 && aligned16(logits)) {
        if (!tile_grid(total / 4, &grid)) return 1;
        hipLaunchKernelGGL(tile_add_mask_kernel<4>, dim3(grid), dim3(256), 0, s, p, total / 4);
    } else {
        if (!tile_grid(total, &grid)) return 1;
        hipLaunchKernelGGL(tile_add_mask_kernel<1>, dim3(grid), dim3(256), 0, s, p, total);
    }
    return tile_launched();
}

int flame_sdpa_softmax_from_lse_tile(const float* logits, const float* lse_row, void* probs_bf16, int BH, int q_t, int k_t,
                                     void* stream) {
    if (BH < 0 || q_t < 0 || k_t < 0) return 1;
    const int64_t total = (int64_t)BH * q_t * k_t;
    if (total == 0) return 0;
    if (!logits || !lse_row || !probs_bf16) return 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint16_t* probs = static_cast<uint16_t*>(probs_bf16);
    unsigned grid;
    if (k_t % 8 == 0 && aligned16(logits) && aligned16(probs_bf16)) {
        if (!tile_grid(total / 8, &grid)) return 1;
        hipLaunchKernelGGL(tile_softmax_from_lse_kernel<8>, dim3(grid), dim3(256), 0, s, logits, lse_row, probs, total / 8, k_t);
    } else {
        if (!tile_grid(total, &grid)) return 1;
        hipLaunchKernelGGL(tile_softmax_from_lse_kernel<1>, dim3(grid), dim3(256), 0, s, logits, lse_row, probs, total, k_t);
    }
    return tile_launched();
}

int flame_sdpa_lse_from_logits_tile(const float* logits, float* out_lse_row, int BH, int q_t, int k_t, void* stream) {
    if (BH < 0 || q_t < 0 || k_t < 0) return 1;
    const int64_t rows = (int64_t)BH * q_t;
    if (rows == 0) return 0;
    if (!out_lse_row || (!logits && k_t > 0)) return 1;
    unsigned grid;
    if (!tile_grid(rows * 64, &grid)) return 1;
    hipLaunchKernelGGL(tile_lse_from_logits_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), logits,
                       out_lse_row, rows, k_t);
    return tile_launched();
}

int flame_sdpa_lse_merge_rows(float* lse_row, const float* tile_lse_row, int BH, int q_t, void* stream) {
    if (BH < 0 || q_t < 0) return 1;
    const int64_t n = (int64_t)BH * q_t;
    if (n == 0) return 0;
    if (!lse_row || !tile_lse_row) return 1;
    unsigned grid;
    if (!tile_grid(n, &grid)) return 1;
    hipLaunchKernelGGL(tile_lse_merge_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), lse_row, tile_lse_row, n);
    return tile_launched();
}

int flame_sdpa_dropout_bf16_inplace(void* probs_bf16, float p, uint64_t seed, int BH, int q_t, int k_t, void* stream) {
    if (BH < 0 || q_t < 0 || k_t < 0) return 1;
    const int64_t total = (int64_t)BH * q_t * k_t;
    if (total == 0) return 0;
    if (!probs_bf16) return 1;
    const float keep = 1.0f - p;
    const float scale = keep > 0.0f ? 1.0f / keep : 0.0f;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint16_t* probs = static_cast<uint16_t*>(probs_bf16);
    unsigned grid;
    if (k_t % 8 == 0 && aligned16(probs_bf16)) {
        if (!tile_grid(total / 8, &grid)) return 1;
        hipLaunchKernelGGL(tile_dropout_kernel<8>, dim3(grid), dim3(256), 0, s, probs, p, scale, seed, total / 8, q_t, k_t);
    } else {
        if (!tile_grid(total, &grid)) return 1;
        hipLaunchKernelGGL(tile_dropout_kernel<1>, dim3(grid), dim3(256), 0, s, probs, p, scale, seed, total, q_t, k_t);
    }
    return tile_launched();
}

// ---- FP8 E4M3 form of saved activations for the offload pool (src/cuda/fp8_quant.cu:74-92, fp8_dequant.cu:42-58)
static float fp8_flushed(float s) { return fabsf(s) < 1.17549435e-38f ? copysignf(0.f, s) : s; }   // the reference's multiply flushes denormal operands
static unsigned fp8_grid(size_t n, bool vec) {
    const size_t work = vec ? (n / 16 > n % 16 ? n / 16 : n % 16) : n;      // lanes that have something to do
    const size_t g = (work + 255) / 256;
    const size_t cap = (size_t)device_cu_count() * 8;                               // grid-stride beyond 8 workgroups per CU
    return (unsigned)(g < 1 ? 1 : g > cap ? cap : g);
}

int flame_bf16_to_fp8(const void* input, void* output, float inv_scale, size_t n_elements, void* stream) {
    if (n_elements == 0) return 0;
    if (!input || !output) return (int)hipErrorInvalidValue;
    const bool vec = aligned16(input) && aligned16(output) && n_elements >= 16;
    const Fp8Params p{input, output, fp8_flushed(inv_scale), n_elements};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (vec) hipLaunchKernelGGL(bf16_to_fp8_kernel<true>, dim3(fp8_grid(n_elements, true)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(bf16_to_fp8_kernel<false>, dim3(fp8_grid(n_elements, false)), dim3(256), 0, s, p);
    return (int)hipGetLastError();
}

int flame_fp8_to_bf16(const void* input, void* output, float scale, size_t n_elements, void* stream) {
    if (n_elements == 0) return 0;
    if (!input || !output) return (int)hipErrorInvalidValue;
    const bool vec = aligned16(input) && aligned16(output) && n_elements >= 16;
    const Fp8Params p{input, output, fp8_flushed(scale), n_elements};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (vec) hipLaunchKernelGGL(fp8_to_bf16_kernel<true>, dim3(fp8_grid(n_elements, true)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(fp8_to_bf16_kernel<false>, dim3(fp8_grid(n_elements, false)), dim3(256), 0, s, p);
    return (int)hipGetLastError();
}

#ifndef FLAME_ATTN_HIPCC_VERSION
#define FLAME_ATTN_HIPCC_VERSION "unknown"
#endif
}  // extern "C"

// ------------------------------------------------------------------------------------------------
// The materialised path (materialised.hpp): rocBLAS GEMMs around the element-wise kernels.  rocBLAS is
// loaded on first use (dlopen), so the library itself links against the HIP runtime only and nothing of
// rocBLAS is touched unless one of these two entry points runs.
// ------------------------------------------------------------------------------------------------
namespace {

struct RocblasApi {
    // rocblas_status f(...): 0 is success
    int (*create_handle)(void** handle) = nullptr;
    int (*set_stream)(void* handle, hipStream_t stream) = nullptr;
    int (*set_atomics_mode)(void* handle, int mode) = nullptr;
    int (*gemm_strided_batched_ex)(void* handle, int transA, int transB, int m, int n, int k, const void* alpha, const void* a,
                                   int a_type, int lda, int64_t stride_a, const void* b, int b_type, int ldb, int64_t stride_b,
                                   const void* beta, const void* c, int c_type, int ldc, int64_t stride_c, void* d, int d_type,
                                   int ldd, int64_t stride_d, int batch_count, int compute_type, int algo, int32_t solution_index,
                                   uint32_t flags) = nullptr;
    void* handle[64] = {};
    bool tried = false, ok = false;
    std::mutex mu;
};
RocblasApi g_rocblas;
// values of rocblas-types.h
constexpr int kOpN = 111, kOpT = 112, kF32 = 151, kBf16 = 168;

int rocblas_for_device(void** handle_out) {
    std::lock_guard<std::mutex> g(g_rocblas.mu);
    if (!g_rocblas.tried) {
        g_rocblas.tried = true;
        void* lib = dlopen("librocblas.so.5", RTLD_NOW | RTLD_LOCAL);
        if (!lib) lib = dlopen("librocblas.so", RTLD_NOW | RTLD_LOCAL);
        if (lib) {
            g_rocblas.create_handle = reinterpret_cast<decltype(g_rocblas.create_handle)>(dlsym(lib, "rocblas_create_handle"));
            g_rocblas.set_stream = reinterpret_cast<decltype(g_rocblas.set_stream)>(dlsym(lib, "rocblas_set_stream"));
            g_rocblas.set_atomics_mode = reinterpret_cast<decltype(g_rocblas.set_atomics_mode)>(dlsym(lib, "rocblas_set_atomics_mode"));
            g_rocblas.gemm_strided_batched_ex =
                reinterpret_cast<decltype(g_rocblas.gemm_strided_batched_ex)>(dlsym(lib, "rocblas_gemm_strided_batched_ex"));
            g_rocblas.ok = g_rocblas.create_handle && g_rocblas.set_stream && g_rocblas.gemm_strided_batched_ex;
        }
    }
    if (!g_rocblas.ok) return FLAME_ATTN_ERR_UNSUPPORTED;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (!g_rocblas.handle[dev]) {
        void* h = nullptr;
        if (g_rocblas.create_handle(&h) != 0 || !h) return FLAME_ATTN_ERR_UNSUPPORTED;
        if (g_rocblas.set_atomics_mode) (void)g_rocblas.set_atomics_mode(h, 0);      // no atomics: the same sums every run
        g_rocblas.handle[dev] = h;
    }
    *handle_out = g_rocblas.handle[dev];
    return FLAME_ATTN_OK;
}

// D[m x n] (column-major, leading dimension ldd) = alpha op(A) op(B) + beta D, batched over the heads of one batch element
int mat_gemm(void* handle, int ta, int tb, int m, int n, int k, float alpha, const void* a, int lda, int64_t sa, const void* b, int ldb,
             int64_t sb, float beta, void* d, int d_type, int ldd, int64_t sd, int batch) {
    const int rc = g_rocblas.gemm_strided_batched_ex(handle, ta, tb, m, n, k, &alpha, a, kBf16, lda, sa, b, kBf16, ldb, sb, &beta, d,
                                                     d_type, ldd, sd, d, d_type, ldd, sd, batch, kF32, 0, 0, 0);
    return rc == 0 ? FLAME_ATTN_OK : FLAME_ATTN_ERR_UNSUPPORTED;
}

int check_view_any_d(const void* base, const int64_t* st) {
    if (!base || !st) return FLAME_ATTN_ERR_INVALID;
    if (st[3] != 1) return FLAME_ATTN_ERR_UNSUPPORTED;
    if (st[0] < 0 || st[1] < 0 || st[2] <= 0 || st[2] > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    return FLAME_ATTN_OK;
}

// bytes per query row of a band: fp32 logits + bf16 P (+ bf16 dS in the backward), over all (batch, head) slices
size_t mat_band_row_bytes(int B, int H, int N_kv, bool backward) { return (size_t)B * H * N_kv * (backward ? 8 : 6); }
size_t mat_fixed_bytes(int B, int H, int N_q, bool backward) { return backward ? align_up((size_t)B * H * N_q * sizeof(float), 256) : 0; }
size_t mat_accum_bytes(int B, int H, int N_kv, int D, int Dv) { return align_up((size_t)B * H * N_kv * (size_t)(D + Dv) * sizeof(float), 256); }

struct MatPlan {
    int tq = 0;              // query rows per band
    bool accumulate = false; // more than one band in the backward: dK / dV are summed in fp32 and stored at the end
    char* rows = nullptr;    // delta [BH, Sq] (backward)
    char* accum = nullptr;   // fp32 dK [BH, Sk, D] then dV [BH, Sk, Dv] (backward, several bands)
    char* scores = nullptr;  // fp32 [BH, tq, Sk]
    char* probs = nullptr;   // bf16 [BH, tq, Sk]
    char* ds = nullptr;      // bf16 [BH, tq, Sk] (backward)
};

// Lays the workspace out for the largest band that fits (whole problem if it does), or fails when not even 16 rows do.
int mat_plan(void* workspace, size_t bytes, int B, int H, int N_q, int N_kv, int D, int Dv, bool backward, MatPlan* out) {
    if (!workspace || !aligned16(workspace)) return FLAME_ATTN_ERR_INVALID;
    char* base = static_cast<char*>(workspace);
    const size_t fixed = mat_fixed_bytes(B, H, N_q, backward), per_row = mat_band_row_bytes(B, H, N_kv, backward);
    constexpr size_t kSlack = 1024;          // alignment of the three band buffers
    if (bytes < fixed + kSlack) return FLAME_ATTN_ERR_INVALID;
    MatPlan p;
    p.rows = base;
    size_t avail = bytes - fixed;
    if (avail >= per_row * (size_t)N_q + kSlack) {
        p.tq = N_q;
    } else {
        if (backward) {
            const size_t acc = mat_accum_bytes(B, H, N_kv, D, Dv);
            if (avail < acc + kSlack) return FLAME_ATTN_ERR_INVALID;
            p.accumulate = true;
            p.accum = base + fixed;
            avail -= acc;
        }
        const size_t rows = (avail - kSlack) / per_row;
        if (rows < 16) return FLAME_ATTN_ERR_INVALID;
        p.tq = (int)std::min<size_t>(rows / 16 * 16, (size_t)N_q);
    }
    char* band = base + fixed + (p.accumulate ? mat_accum_bytes(B, H, N_kv, D, Dv) : 0);
    const size_t n = (size_t)B * H * p.tq * N_kv;
    p.scores = band;
    p.probs = band + align_up(n * 4, 256);
    p.ds = p.probs + align_up(n * 2, 256);
    *out = p;
    return FLAME_ATTN_OK;
}

void mat_fill_mask(MaskArgs& m, int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                   const void* bias, int bias_dtype, const int64_t* bias_strides, int mask_mode = kMaskU8) {
    m.kv_len = kv_len;
    m.mask = keep_mask;
    m.mask_mode = mask_mode;
    m.sb = keep_mask ? mask_strides[0] : 0;
    m.sh = keep_mask ? mask_strides[1] : 0;
    m.sq = keep_mask ? mask_strides[2] : 0;
    m.sk = keep_mask ? mask_strides[3] : 0;
    m.causal = causal ? 1 : 0;
    m.bias = bias;
    if (bias) {
        m.bb = bias_strides[0]; m.bh = bias_strides[1]; m.bq = bias_strides[2]; m.bk = bias_strides[3];
        m.bias_f32 = bias_dtype == FLAME_ATTN_DTYPE_F32;
    }
}

}  // namespace

extern "C" {

size_t flame_attn_materialised_workspace_bytes(int B, int H, int N_q, int N_kv, int D, int Dv, int backward) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0 || Dv <= 0) return 0;
    const bool bw = backward != 0;
    const size_t fixed = mat_fixed_bytes(B, H, N_q, bw), per_row = mat_band_row_bytes(B, H, N_kv, bw);
    const size_t whole = fixed + per_row * ((size_t)N_q + 1) + 1024;
    // bands of at least 64 rows and at most 512 MiB, with the fp32 dK / dV sums a banded backward needs
    const size_t band_rows = std::max<size_t>(64, std::min<size_t>((size_t)N_q, ((size_t)512 << 20) / per_row / 16 * 16));
    const size_t banded = fixed + (bw ? mat_accum_bytes(B, H, N_kv, D, Dv) : 0) + per_row * (band_rows + 1) + 1024;
    return std::min(whole, banded);
}

static int mat_fwd_impl(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                        const void* bias, int bias_dtype, const int64_t* bias_strides,
                        void* workspace, size_t workspace_bytes, void* stream, int mask_mode,
                        float dropout_p, uint64_t dropout_seed, int draw_cq, int draw_ck) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0 || Dv <= 0) return FLAME_ATTN_ERR_INVALID;
    if (!(scale > 0.f) || !isfinite(scale)) return FLAME_ATTN_ERR_INVALID;
    int rc;
    if ((rc = check_view_any_d(Q, q_strides)) || (rc = check_view_any_d(K, k_strides)) || (rc = check_view_any_d(V, v_strides)) ||
        (rc = check_view_any_d(O, o_strides)))
        return rc;
    if ((keep_mask && !mask_strides) || (bias && !bias_strides)) return FLAME_ATTN_ERR_INVALID;
    if (bias && bias_dtype != FLAME_ATTN_DTYPE_BF16 && bias_dtype != FLAME_ATTN_DTYPE_F32) return FLAME_ATTN_ERR_INVALID;
    if ((int64_t)B * H * N_q > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    MatPlan plan;
    if ((rc = mat_plan(workspace, workspace_bytes, B, H, N_q, N_kv, D, Dv, false, &plan))) return rc;
    void* handle = nullptr;
    if ((rc = rocblas_for_device(&handle))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> enqueue(g_rocblas.mu);          // the handle's stream is set per call
    if (g_rocblas.set_stream(handle, s) != 0) return FLAME_ATTN_ERR_UNSUPPORTED;
    const uint16_t* q = static_cast<const uint16_t*>(Q) + q_off;
    const uint16_t* k = static_cast<const uint16_t*>(K) + k_off;
    const uint16_t* v = static_cast<const uint16_t*>(V) + v_off;
    uint16_t* o = static_cast<uint16_t*>(O) + o_off;
    MatRowsParams rp;
    rp.scores = reinterpret_cast<float*>(plan.scores);
    rp.probs = reinterpret_cast<uint16_t*>(plan.probs);
    rp.lse = LSE ? static_cast<float*>(LSE) + lse_off : nullptr;
    rp.H = H; rp.Sq = N_q; rp.Sk = N_kv;
    rp.from_lse = 0;
    mat_fill_mask(rp.m, causal, kv_len, keep_mask, mask_strides, bias, bias_dtype, bias_strides, mask_mode);
    if (dropout_p != 0.f) {
        if (!set_dropout(rp.m, dropout_p, dropout_seed, draw_cq, draw_ck, N_q, N_kv)) return FLAME_ATTN_ERR_INVALID;
        rp.dropout = 1;
    }
    for (int q0 = 0; q0 < N_q; q0 += plan.tq) {
        const int tq = std::min(plan.tq, N_q - q0);
        const int64_t band = (int64_t)tq * N_kv;
        for (int b = 0; b < B; ++b) {       // S^T [Sk x tq] = scale K Q^T, all heads of one batch element per call
            rc = mat_gemm(handle, kOpT, kOpN, N_kv, tq, D, scale, k + b * k_strides[0], (int)k_strides[2], k_strides[1],
                          q + b * q_strides[0] + (int64_t)q0 * q_strides[2], (int)q_strides[2], q_strides[1], 0.f,
                          rp.scores + (int64_t)b * H * band, kF32, N_kv, band, H);
            if (rc) return rc;
        }
        rp.tq = tq; rp.q0 = q0;
        hipLaunchKernelGGL(mat_rows_kernel, dim3((unsigned)((int64_t)B * H * tq)), dim3(256), 0, s, rp);
        for (int b = 0; b < B; ++b) {       // O^T [Dv x tq] = V^T P^T
            rc = mat_gemm(handle, kOpN, kOpN, Dv, tq, N_kv, 1.f, v + b * v_strides[0], (int)v_strides[2], v_strides[1],
                          rp.probs + (int64_t)b * H * band, N_kv, band, 0.f, o + b * o_strides[0] + (int64_t)q0 * o_strides[2], kBf16,
                          (int)o_strides[2], o_strides[1], H);
            if (rc) return rc;
        }
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

int flame_attn_fwd_materialised_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                     int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                                     const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                     const int64_t* o_strides,
                                     int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                     int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                     const void* bias, int bias_dtype, const int64_t* bias_strides,
                                     float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    return mat_fwd_impl(Q, K, V, O, LSE, B, H, N_q, N_kv, D, Dv, scale, q_strides, k_strides, v_strides, o_strides, q_off, k_off,
                        v_off, o_off, lse_off, causal, kv_len, keep_mask, mask_strides, bias, bias_dtype, bias_strides, workspace,
                        workspace_bytes, stream, kMaskU8, dropout_p, dropout_seed, draw_chunk_q, draw_chunk_kv);
}

int flame_attn_bwd_materialised_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                     const void* LSE, void* dQ, void* dK, void* dV,
                                     int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                                     const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                     const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                     const int64_t* dk_strides, const int64_t* dv_strides,
                                     int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                     int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                     int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                     float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0 || Dv <= 0) return FLAME_ATTN_ERR_INVALID;
    if (!(scale > 0.f) || !isfinite(scale) || !LSE) return FLAME_ATTN_ERR_INVALID;
    int rc;
    if ((rc = check_view_any_d(Q, q_strides)) || (rc = check_view_any_d(K, k_strides)) || (rc = check_view_any_d(V, v_strides)) ||
        (rc = check_view_any_d(O, o_strides)) || (rc = check_view_any_d(dO, do_strides)) || (rc = check_view_any_d(dQ, dq_strides)) ||
        (rc = check_view_any_d(dK, dk_strides)) || (rc = check_view_any_d(dV, dv_strides)))
        return rc;
    if (keep_mask && !mask_strides) return FLAME_ATTN_ERR_INVALID;
    if ((int64_t)B * H * N_q > 0x7fffffff) return FLAME_ATTN_ERR_UNSUPPORTED;
    MatPlan plan;
    if ((rc = mat_plan(workspace, workspace_bytes, B, H, N_q, N_kv, D, Dv, true, &plan))) return rc;
    void* handle = nullptr;
    if ((rc = rocblas_for_device(&handle))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> enqueue(g_rocblas.mu);
    if (g_rocblas.set_stream(handle, s) != 0) return FLAME_ATTN_ERR_UNSUPPORTED;
    const uint16_t* q = static_cast<const uint16_t*>(Q) + q_off;
    const uint16_t* k = static_cast<const uint16_t*>(K) + k_off;
    const uint16_t* v = static_cast<const uint16_t*>(V) + v_off;
    const uint16_t* d_o = static_cast<const uint16_t*>(dO) + do_off;
    uint16_t* dq = static_cast<uint16_t*>(dQ) + dq_off;
    uint16_t* dk = static_cast<uint16_t*>(dK) + dk_off;
    uint16_t* dv = static_cast<uint16_t*>(dV) + dv_off;
    float* delta = reinterpret_cast<float*>(plan.rows);
    {
        MatDeltaParams dp;
        dp.o = static_cast<const uint16_t*>(O) + o_off;
        dp.dout = d_o;
        dp.os = mk(o_strides); dp.dos = mk(do_strides);
        dp.delta = delta;
        dp.B = B; dp.H = H; dp.Sq = N_q; dp.dv = Dv;
        const int64_t rows = (int64_t)B * H * N_q;
        hipLaunchKernelGGL(mat_delta_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, dp);
    }
    MatRowsParams rp;
    rp.scores = reinterpret_cast<float*>(plan.scores);
    rp.probs = reinterpret_cast<uint16_t*>(plan.probs);
    rp.lse = const_cast<float*>(static_cast<const float*>(LSE) + lse_off);
    rp.H = H; rp.Sq = N_q; rp.Sk = N_kv;
    rp.from_lse = 1;
    mat_fill_mask(rp.m, causal, kv_len, keep_mask, mask_strides, nullptr, FLAME_ATTN_DTYPE_F32, nullptr);
    MaskArgs drop = rp.m;            // drop_thr = 0: no dropout
    if (dropout_p != 0.f && !set_dropout(drop, dropout_p, dropout_seed, draw_chunk_q, draw_chunk_kv, N_q, N_kv)) return FLAME_ATTN_ERR_INVALID;
    uint16_t* ds = reinterpret_cast<uint16_t*>(plan.ds);
    float* acc_dk = reinterpret_cast<float*>(plan.accum);
    float* acc_dv = plan.accum ? acc_dk + (size_t)B * H * N_kv * D : nullptr;
    for (int q0 = 0; q0 < N_q; q0 += plan.tq) {
        const int tq = std::min(plan.tq, N_q - q0);
        const int64_t band = (int64_t)tq * N_kv;
        const float beta = (plan.accumulate && q0 > 0) ? 1.f : 0.f;
        for (int b = 0; b < B; ++b) {       // S^T = scale K Q^T
            rc = mat_gemm(handle, kOpT, kOpN, N_kv, tq, D, scale, k + b * k_strides[0], (int)k_strides[2], k_strides[1],
                          q + b * q_strides[0] + (int64_t)q0 * q_strides[2], (int)q_strides[2], q_strides[1], 0.f,
                          rp.scores + (int64_t)b * H * band, kF32, N_kv, band, H);
            if (rc) return rc;
        }
        rp.tq = tq; rp.q0 = q0;
        hipLaunchKernelGGL(mat_rows_kernel, dim3((unsigned)((int64_t)B * H * tq)), dim3(256), 0, s, rp);      // P = exp(S - LSE)
        for (int b = 0; b < B; ++b) {       // dP^T [Sk x tq] = V dO^T, into the logits' buffer (P has been formed)
            rc = mat_gemm(handle, kOpT, kOpN, N_kv, tq, Dv, 1.f, v + b * v_strides[0], (int)v_strides[2], v_strides[1],
                          d_o + b * do_strides[0] + (int64_t)q0 * do_strides[2], (int)do_strides[2], do_strides[1], 0.f,
                          rp.scores + (int64_t)b * H * band, kF32, N_kv, band, H);
            if (rc) return rc;
        }
        {
            const int64_t n = (int64_t)B * H * band;
            hipLaunchKernelGGL(mat_ds_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, rp.probs, rp.scores, delta, ds, n, N_kv,
                               tq, N_q, q0, drop);
        }
        for (int b = 0; b < B; ++b) {
            const uint16_t* pb = rp.probs + (int64_t)b * H * band;
            const uint16_t* dsb = ds + (int64_t)b * H * band;
            // dV^T [Dv x Sk] (+)= dO^T P ; dK^T [D x Sk] (+)= scale Q^T dS ; dQ^T [D x tq] = scale K^T dS^T
            if (plan.accumulate) {
                rc = mat_gemm(handle, kOpN, kOpT, Dv, N_kv, tq, 1.f, d_o + b * do_strides[0] + (int64_t)q0 * do_strides[2],
                              (int)do_strides[2], do_strides[1], pb, N_kv, band, beta, acc_dv + (size_t)b * H * N_kv * Dv, kF32, Dv,
                              (int64_t)N_kv * Dv, H);
                if (rc) return rc;
                rc = mat_gemm(handle, kOpN, kOpT, D, N_kv, tq, scale, q + b * q_strides[0] + (int64_t)q0 * q_strides[2], (int)q_strides[2],
                              q_strides[1], dsb, N_kv, band, beta, acc_dk + (size_t)b * H * N_kv * D, kF32, D, (int64_t)N_kv * D, H);
                if (rc) return rc;
            } else {
                rc = mat_gemm(handle, kOpN, kOpT, Dv, N_kv, tq, 1.f, d_o + b * do_strides[0], (int)do_strides[2], do_strides[1], pb, N_kv,
                              band, 0.f, dv + b * dv_strides[0], kBf16, (int)dv_strides[2], dv_strides[1], H);
                if (rc) return rc;
                rc = mat_gemm(handle, kOpN, kOpT, D, N_kv, tq, scale, q + b * q_strides[0], (int)q_strides[2], q_strides[1], dsb, N_kv,
                              band, 0.f, dk + b * dk_strides[0], kBf16, (int)dk_strides[2], dk_strides[1], H);
                if (rc) return rc;
            }
            rc = mat_gemm(handle, kOpN, kOpN, D, tq, N_kv, scale, k + b * k_strides[0], (int)k_strides[2], k_strides[1], dsb, N_kv, band, 0.f,
                          dq + b * dq_strides[0] + (int64_t)q0 * dq_strides[2], kBf16, (int)dq_strides[2], dq_strides[1], H);
            if (rc) return rc;
        }
    }
    if (plan.accumulate) {
        const int64_t nk = (int64_t)B * H * N_kv * D, nv = (int64_t)B * H * N_kv * Dv;
        hipLaunchKernelGGL(mat_store_kernel, dim3((unsigned)((nk + 255) / 256)), dim3(256), 0, s, acc_dk, dk, mk(dk_strides), H, N_kv, D, nk);
        hipLaunchKernelGGL(mat_store_kernel, dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, s, acc_dv, dv, mk(dv_strides), H, N_kv, Dv, nv);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLAME_ATTN_OK : (int)e;
}

// names the compiler that built this library: the static checks of the hand-emitted instructions are
// only meaningful for the assembly that this very compiler generates
const char* flame_attn_version(void) { return "flame-attn-gfx950 0.2 (hipcc " FLAME_ATTN_HIPCC_VERSION ")"; }

}  // extern "C"
