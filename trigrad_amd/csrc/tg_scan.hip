// tg_scan.hip -- single-pass exclusive prefix sum of uint32 with decoupled look-back.
//
// HBM-bound: 4 B read + 4 B written per element, one pass.  A workgroup of
// 512 threads owns a tile of 2048 elements (one 16-byte load per thread).
// Inside a wave the scan runs on DPP row shifts and row broadcasts (wave64);
// the tile prefix comes from the predecessors' published state words, read by
// one wave, 64 predecessors per step.
//
// State word (one uint64 per tile): bits 63..62 = 0 not ready, 1 tile aggregate
// ready, 2 inclusive prefix ready; bits 31..0 = the value.  Value and flag
// share one word, so relaxed agent-scope atomic loads/stores are sufficient.
// Tiles are numbered by an atomic ticket taken at workgroup start, so every
// tile a workgroup waits for is already running; a grid that fits the device
// at once uses the workgroup ids instead.  The wait is bounded: on
// expiry the kernel records TG_STATUS_LOOKBACK_TIMEOUT and carries on (with a
// wrong result) so that every wave still exits.
#include <mutex>

#include "tg_scan.hpp"

namespace tg {

__global__ void scan_init_kernel(uint32_t *ticket, uint64_t *states, int n_tiles, uint32_t *total, uint32_t *status) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) {
        *ticket = 0;
        *total = 0;
        if (status) *status = TG_STATUS_OK;
    }
    if (i < n_tiles) states[i] = 0;
}

__global__ __launch_bounds__(kScanThreads) void scan_lookback_kernel(const uint32_t *__restrict__ in, uint32_t *out, int64_t n,
                                                                     uint32_t *total, uint32_t *ticket, uint64_t *states,
                                                                     int n_tiles, uint32_t *status, uint32_t head_stride,
                                                                     uint32_t head_capacity, uint32_t *__restrict__ heads) {
    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_wave_total[kScanThreads / kWave];
    __shared__ uint32_t s_tile_prefix;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    if (tid == 0) s_tile = ticket ? atomicAdd(ticket, 1u) : blockIdx.x;  // no ticket: the whole grid is resident
    __syncthreads();
    const int tile = (int)s_tile;

    const int64_t base = (int64_t)tile * kScanTile + (int64_t)tid * 4;
    uint32_t x[4] = {0, 0, 0, 0};
    if (base + 4 <= n) {
        uint4 v = *reinterpret_cast<const uint4 *>(in + base);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else {
        for (int k = 0; k < 4; k++)
            if (base + k < n) x[k] = in[base + k];
    }
    const uint32_t thread_sum = x[0] + x[1] + x[2] + x[3];
    const uint32_t incl = wave_inclusive_scan_u32(thread_sum);
    if (lane == kWave - 1) s_wave_total[wave] = incl;
    __syncthreads();

    if (wave == 0) {
        // scan of the wave totals, then publish and look back
        uint32_t wt = (lane < kScanThreads / kWave) ? s_wave_total[lane] : 0u;
        uint32_t wincl = wave_inclusive_scan_u32(wt);
        uint32_t tile_total = (uint32_t)__builtin_amdgcn_readlane((int)wincl, kScanThreads / kWave - 1);
        if (lane < kScanThreads / kWave) s_wave_total[lane] = wincl - wt;  // exclusive wave offsets

        const uint32_t prefix = scan_tile_prefix(states, tile, tile_total, n_tiles, total, status);
        if (lane == 0) s_tile_prefix = prefix;
    }
    __syncthreads();

    uint32_t run = s_tile_prefix + s_wave_total[wave] + (incl - thread_sum);
    uint32_t y[4];
    for (int k = 0; k < 4; k++) { y[k] = run; run += x[k]; }
    if (heads) {
        // element i owns the output positions [y, y + x): note for every multiple of
        // head_stride which element owns it (few elements own one, most own none)
        for (int k = 0; k < 4; k++) {
            if (x[k] == 0 || base + k >= n) continue;
            const uint32_t first = (y[k] + head_stride - 1) / head_stride, last = (y[k] + x[k] - 1) / head_stride;
            for (uint32_t h = first; h <= last && h < head_capacity; h++) heads[h] = (uint32_t)(base + k);
        }
    }
    if (base + 4 <= n) {
        *reinterpret_cast<uint4 *>(out + base) = make_uint4(y[0], y[1], y[2], y[3]);
    } else {
        for (int k = 0; k < 4; k++)
            if (base + k < n) out[base + k] = y[k];
    }
}

}  // namespace tg

using namespace tg;

static size_t scan_state_offset() { return 64; }  // ticket lives in the first 64 bytes

extern "C" size_t tg_scan_workspace_bytes(int64_t n) {
    if (n < 0) return 0;
    int64_t tiles = ceil_div64(n, kScanTile);
    if (tiles < 1) tiles = 1;
    return scan_state_offset() + (size_t)tiles * sizeof(uint64_t);
}

// Argument checks and launches shared by the two entry points; `workspace` holds at least
// tg_scan_workspace_bytes(n) bytes, 8-byte aligned.
static int scan_run(const char *fn, const uint32_t *in, uint32_t *out, int64_t n, uint32_t *total, void *workspace,
                    uint32_t *status, uint32_t head_stride, uint32_t head_capacity, uint32_t *heads, hipStream_t s) {
    if (n < 0 || !total || !workspace || (n > 0 && (!in || !out))) {
        set_error("%s: null pointer or negative size", fn);
        return TG_E_ARG;
    }
    if (((uintptr_t)in & 15) || ((uintptr_t)out & 15) || ((uintptr_t)workspace & 7)) {
        set_error("%s: in/out must be 16-byte aligned, workspace 8-byte aligned", fn);
        return TG_E_ARG;
    }
    if (heads && head_stride == 0) {
        set_error("%s: head_stride must be positive when heads is given", fn);
        return TG_E_ARG;
    }
    if (n > (int64_t)kScanTile * 0x7fffffff / 2) {
        set_error("%s: n too large", fn);
        return TG_E_ARG;
    }
    const int n_tiles = (int)ceil_div64(n, kScanTile);
    uint32_t *ticket = (uint32_t *)workspace;
    uint64_t *states = (uint64_t *)((char *)workspace + scan_state_offset());
    const int init_blocks = n_tiles > 0 ? ceil_div(n_tiles, 256) : 1;
    // a kernel, not a memset: the clearing may be recorded into a graph by the caller
    TG_LAUNCH(scan_init_kernel, dim3(init_blocks), dim3(256), 0, s, ticket, states, n_tiles, total, status);
    if (int e = check_launch("scan_init_kernel")) return e;
    if (n_tiles == 0) return 0;
    static int resident_cache[kMaxDevices] = {0};
    if (n_tiles <= resident_workgroups((const void *)scan_lookback_kernel, kScanThreads, resident_cache)) ticket = nullptr;
    TG_LAUNCH(scan_lookback_kernel, dim3(n_tiles), dim3(kScanThreads), 0, s, in, out, n, total, ticket, states,
                       n_tiles, status, head_stride, head_capacity, heads);
    return check_launch("scan_lookback_kernel");
}

extern "C" int tg_scan_exclusive_u32(const uint32_t *in, uint32_t *out, int64_t n, uint32_t *total, void *workspace,
                                     size_t workspace_bytes, uint32_t *status, uint32_t head_stride, uint32_t head_capacity,
                                     uint32_t *heads, void *stream) {
    if (n >= 0 && workspace && workspace_bytes < tg_scan_workspace_bytes(n)) {
        set_error("tg_scan_exclusive_u32: workspace of %zu bytes, need %zu", workspace_bytes, tg_scan_workspace_bytes(n));
        return TG_E_WORKSPACE;
    }
    return scan_run("tg_scan_exclusive_u32", in, out, n, total, workspace, status, head_stride, head_capacity, heads,
                    (hipStream_t)stream);
}

// ---- the same scan for callers that cannot allocate ------------------------------------
// The look-back state (ticket + one word per tile of 2048 elements) lives in a file-scope device array
// instead of a caller's workspace.  Every GPU the library runs on holds its own copy of the array at its
// own address, found once per device with hipGetSymbolAddress; host code uses that address only, never the
// array's name.  All calls on one GPU share the array: calls that overlap there (two streams, two
// threads) race.  scan_init_kernel clears the part a call uses before the scan reads it.
constexpr int64_t kStaticScanMaxN = TG_SCAN_NOALLOC_MAX_N;
constexpr size_t kStaticScanBytes = 64 + (size_t)(kStaticScanMaxN / kScanTile) * sizeof(uint64_t);
static_assert(kStaticScanMaxN % kScanTile == 0, "whole tiles");
static __device__ __align__(256) unsigned char scratch[kStaticScanBytes];

// -> the array's address on the current device, or nullptr with *error = the runtime's error code.
static void *static_scan_workspace(int *error) {
    static std::mutex mutex;
    static void *address[kMaxDevices] = {nullptr};
    int dev = -1;
    const hipError_t have_device = hipGetDevice(&dev);
    if (have_device != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        set_error("tg_scan_exclusive_u32_noalloc: no current device");
        *error = have_device != hipSuccess ? (int)have_device : (int)hipErrorInvalidDevice;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (!address[dev]) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            (void)hipGetLastError();
            set_error("tg_scan_exclusive_u32_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
            *error = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
            return nullptr;
        }
        address[dev] = ptr;
    }
    return address[dev];
}

extern "C" int64_t tg_scan_noalloc_max_n(void) { return kStaticScanMaxN; }

extern "C" int tg_scan_exclusive_u32_noalloc(const uint32_t *in, uint32_t *out, int64_t n, uint32_t *total, uint32_t *status,
                                             uint32_t head_stride, uint32_t head_capacity, uint32_t *heads, void *stream) {
    if (n > kStaticScanMaxN) {
        set_error("tg_scan_exclusive_u32_noalloc: n = %lld exceeds the %lld elements the built-in state covers; "
                  "use tg_scan_exclusive_u32 with a workspace", (long long)n, (long long)kStaticScanMaxN);
        return TG_E_ARG;
    }
    int runtime_error = 0;
    void *workspace = static_scan_workspace(&runtime_error);
    if (!workspace) return runtime_error;  // a hipError_t: the arguments were not at fault
    return scan_run("tg_scan_exclusive_u32_noalloc", in, out, n, total, workspace, status, head_stride, head_capacity, heads,
                    (hipStream_t)stream);
}
