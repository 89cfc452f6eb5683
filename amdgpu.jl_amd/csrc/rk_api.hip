// C ABI entry points of librk.so: argument validation (runs without a GPU), dispatch on the
// element types, workspace management.  The kernels live in rk_*_impl.hpp / rk_*.hip.
#include <atomic>
#include <mutex>
#include <cstdlib>
#include <cstddef>
#include <cstring>

#include "rk_common.hpp"
#include "rk_reduce_impl.hpp"
#include "rk_scan_impl.hpp"

namespace rk {

const DeviceInfo& device_info() {
    static DeviceInfo info[64];
    static std::atomic<int> ready[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!ready[dev].load(std::memory_order_acquire)) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        info[dev].cus = cus;      // benign race: every writer stores the same value
        ready[dev].store(1, std::memory_order_release);
    }
    return info[dev];
}

static int env_int(const char* name, int dflt, int lo, int hi) {
    const char* s = std::getenv(name);
    if (!s || !*s) return dflt;
    const long v = std::strtol(s, nullptr, 10);
    if (v < lo || v > hi) return dflt;
    return (int)v;
}

// Workgroups per compute unit the multi-workgroup reductions aim for (RK_REDUCE_BLOCKS_PER_CU).
// Measured on MI355X for the full Float32 sum of 2^28 elements: 1 -> 5.9, 2 -> 7.0, 4 -> 6.9, 8 -> 6.8,
// 32 -> 6.7 TB/s: two persistent workgroups per unit keep enough loads in flight, more only lengthen the fold.
int tune_reduce_blocks_per_cu() {
    static const int v = env_int("RK_REDUCE_BLOCKS_PER_CU", 2, 1, 64);
    return v;
}

// Workgroups per compute unit of the lanes-along-inner reduction (RK_REDUCE_STRIDED_BLOCKS_PER_CU).
// Measured for mapreduce(abs2, +, 8192 x 8192 Float32; dims=2): 1 -> 5.3, 2 -> 6.5, 4 -> 6.3, 8 -> 6.0 TB/s.
int tune_reduce_strided_blocks_per_cu() {
    static const int v = env_int("RK_REDUCE_STRIDED_BLOCKS_PER_CU", 2, 1, 64);
    return v;
}

// Longest line (bytes) still reduced by one wave; longer lines get a workgroup each (RK_REDUCE_WAVE_MAX_BYTES).
int tune_reduce_wave_max_bytes() {
    static const int v = env_int("RK_REDUCE_WAVE_MAX_BYTES", 8192, 1, 1 << 30);
    return v;
}

// Look-back polling back-off of the scan, in units of 512 clocks (RK_SCAN_BACKOFF).
int tune_scan_backoff() {
    static const int v = env_int("RK_SCAN_BACKOFF", 1, 0, 64);
    return v;
}

// Start-up stagger of the single-pass scan in launch order: the last workgroup of the first resident round starts this
// many ticks of the 100 MHz clock after the first (RK_SCAN_STAGGER_TICKS; 0 = all at once).
int tune_scan_stagger_ticks() {
    static const int v = env_int("RK_SCAN_STAGGER_TICKS", 500, 0, 100000);
    return v;
}

// Tile numbers of the single-pass kernels that run one tile per workgroup (RK_ORDERED_IDS): 0 = from the launch order
// while the whole grid is resident at once and from the device-wide counter beyond that, 1 = always the launch order,
// 2 = always the counter.  Read at every call.
int tune_ordered_ids() {
    return env_int("RK_ORDERED_IDS", 0, 0, 2);
}

// Persistent 256-thread workgroups per compute unit of the look-back scan; larger workgroups scale it
// down (RK_SCAN_BLOCKS_PER_CU).
int tune_scan_blocks_per_cu() {
    static const int v = env_int("RK_SCAN_BLOCKS_PER_CU", 4, 1, 16);
    return v;
}

// Waves per workgroup of the look-back scan: 0 = by line length, else 4, 8 or 16 (RK_SCAN_WAVES).
int tune_scan_waves() {
    static const int v = env_int("RK_SCAN_WAVES", 0, 0, 16);
    return (v == 4 || v == 8 || v == 16) ? v : 0;
}

// 1: the single-pass scan takes its tile ids from a device-wide counter (forward progress whatever the order in which
// workgroups start) instead of from the launch order (RK_SCAN_DYNAMIC_IDS).
int tune_scan_dynamic_ids() {
    static const int v = env_int("RK_SCAN_DYNAMIC_IDS", 0, 0, 1);
    return v;
}

// 0: long lines of 1- and 2-byte integers are scanned in widened tiles of 32 Ki elements instead of packed ones of 128 KiB
// (RK_SCAN_PACKED).
// 0: the tile-a-line scan runs four waves a workgroup whatever the line length (RK_SCAN_TILES_WAVES).
int tune_scan_tiles_waves() {
    static const int v = env_int("RK_SCAN_TILES_WAVES", 1, 0, 1);
    return v;
}

// 0: long lines at odd addresses are scanned by the persistent counter-fed kernel instead of the one in launch order
// (RK_SCAN_ORDERED_UNALIGNED).
int tune_scan_ordered_unaligned() {
    static const int v = env_int("RK_SCAN_ORDERED_UNALIGNED", 1, 0, 1);
    return v;
}

// 0: long lines of 8-byte values are scanned by the persistent counter-fed kernel instead of the one in launch order
// (RK_SCAN_ORDERED8).
int tune_scan_ordered8() {
    static const int v = env_int("RK_SCAN_ORDERED8", 1, 0, 1);
    return v;
}
int tune_scan_packed() {
    static const int v = env_int("RK_SCAN_PACKED", 1, 0, 1);
    return v;
}

// 0: scans across the rows of a wide matrix (few strips of columns) take the three-pass path (totals, scan of the totals,
// scan) instead of the single-pass kernel with look-back (RK_SCAN_ROWS_ORDERED).
int tune_scan_rows_ordered() {
    static const int v = env_int("RK_SCAN_ROWS_ORDERED", 1, 0, 1);
    return v;
}

// 0: scans along the second dim of arrays whose first dim is at most half a strip of columns take the two-pass tiles
// (scan_narrow_kernel) or the strips instead of the single pass with several rows per load (RK_SCAN_ROWS_PACKED).
int tune_scan_rows_packed() {
    static const int v = env_int("RK_SCAN_ROWS_PACKED", 1, 0, 1);
    return v;
}

// Workgroups per compute unit the scan across rows aims for when it cuts the rows into slices
// (RK_SCAN_SLICE_BLOCKS_PER_CU).
int tune_scan_slice_blocks_per_cu() {
    static const int v = env_int("RK_SCAN_SLICE_BLOCKS_PER_CU", 32, 1, 256);
    return v;
}

// Unsuccessful poll rounds one bounded wait may spend before it gives up (RK_WAIT_BUDGET, rk_set_wait_budget).
// A round is one device-coherent load plus the back-off, about a microsecond; correct calls resolve in tens of rounds.
constexpr long long WAIT_BUDGET_DEFAULT = 1ll << 21;
static std::atomic<long long> g_wait_budget{0};
long long wait_budget() {
    long long v = g_wait_budget.load(std::memory_order_relaxed);
    if (v <= 0) {
        const char* s = std::getenv("RK_WAIT_BUDGET");
        v = (s && *s) ? std::strtoll(s, nullptr, 10) : 0;
        if (v <= 0) v = WAIT_BUDGET_DEFAULT;
        g_wait_budget.store(v, std::memory_order_relaxed);
    }
    return v;
}

static bool valid_dtype(int dt) { return dt >= RK_F32 && dt <= RK_U16; }   // unsupported combinations fail in the dispatch

static bool valid_shape(int ndim, const int64_t* shape, int64_t* total) {
    if (ndim < 0 || ndim > RK_MAX_DIMS) return false;
    if (ndim > 0 && shape == nullptr) return false;
    int64_t n = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0) return false;
        if (shape[d] != 0 && n > INT64_MAX / shape[d]) return false;
        n *= shape[d];
    }
    *total = n;
    return true;
}

size_t findall_workspace_need(int64_t n);   // rk_select.hip

// Prepares a workspace: header, tickets and descriptors to zero (tag 0 = never valid), the scan epoch to
// WS_EPOCH_FIRST.  A kernel, not hipMemsetAsync: memset nodes recorded into a captured graph have replayed
// wrongly on this platform, and a fill kernel is safe either way.  64-bit words (what the descriptors are);
// word 0 is the header's scan_counter = epoch << 32.
__global__ __launch_bounds__(256) void workspace_init_kernel(uint64_t* ws, size_t head_words, size_t desc_word0, size_t total_words) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total_words; i += stride) {
        if (i >= head_words && i < desc_word0) continue;          // partials: never read before written
        ws[i] = i == 0 ? (uint64_t)WS_EPOCH_FIRST << 32 : 0ull;
    }
}

static int32_t workspace_init(void* ws, size_t ws_bytes, hipStream_t stream) {
    static_assert(offsetof(WsHeader, scan_counter) == 0 && WS_PARTIALS_OFFSET % 8 == 0 && WS_DESC_OFFSET % 8 == 0, "layout in 64-bit words");
    workspace_init_kernel<<<1024, 256, 0, stream>>>((uint64_t*)ws, WS_PARTIALS_OFFSET / 8, WS_DESC_OFFSET / 8, ws_bytes / 8);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

}  // namespace rk

// ---- bookkeeping of rk_accumulate_static ---------------------------------------------------------------------
// One array per GPU inside the library image.  In host code its name is only a handle for hipGetSymbolAddress;
// the device address obtained there (per device: each GPU holds its own copy) is what kernels and fills receive.
static __device__ __align__(256) unsigned char scratch[RK_STATIC_SCRATCH_BYTES];

namespace rk {
constexpr int STATIC_MAX_DEVICES = 64;
static std::mutex g_static_mutex;
static void* g_static_ptr[STATIC_MAX_DEVICES];      // device address of `scratch` on each device, null until prepared

// Device address of the current device's scratch array, prepared (on `stream`) at the first call on that device.
static int32_t static_scratch(hipStream_t stream, void** out) {
    int dev = 0;
    RK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return RK_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_static_ptr[dev] == nullptr) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        RK_HIP(hipStreamIsCapturing(stream, &cap));
        if (cap != hipStreamCaptureStatusNone) return RK_ERR_WORKSPACE;   // a captured preparation would replay with every graph launch
        void* ptr = nullptr;
        RK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr || !is_aligned(ptr, 256)) return RK_ERR_WORKSPACE;
        const int32_t st = workspace_init(ptr, RK_STATIC_SCRATCH_BYTES, stream);
        if (st != RK_SUCCESS) return st;
        // the array serves every stream of the device from now on: nobody may see it before the fill has finished
        RK_HIP(hipStreamSynchronize(stream));
        g_static_ptr[dev] = ptr;
    }
    *out = g_static_ptr[dev];
    return RK_SUCCESS;
}
}  // namespace rk

using namespace rk;

static int32_t findminmax_dispatch(rk_dtype in, const FindArgs& a) {
    switch (in) {
        case RK_F32: return findminmax_f32(a);
        case RK_F16: return findminmax_f16(a);
        case RK_F64: return findminmax_f64(a);
        case RK_I32: return findminmax_i32(a);
        case RK_I64: return findminmax_i64(a);
        case RK_U8:  return findminmax_u8(a);
        case RK_I8:  return findminmax_i8(a);
        case RK_I16: return findminmax_i16(a);
        case RK_U16: return findminmax_u16(a);
        case RK_U32: return findminmax_u32(a);
        case RK_U64: return findminmax_u64(a);
        default: return RK_ERR_UNSUPPORTED;
    }
}

extern "C" {

int32_t rk_version(void) { return RK_VERSION; }

const char* rk_status_string(int32_t status) {
    switch (status) {
        case RK_SUCCESS: return "RK_SUCCESS";
        case RK_ERR_INVALID_ARGUMENT: return "RK_ERR_INVALID_ARGUMENT: null pointer, bad enum value or rank out of range";
        case RK_ERR_UNSUPPORTED: return "RK_ERR_UNSUPPORTED: combination outside the enumerated op / element-type set";
        case RK_ERR_WORKSPACE: return "RK_ERR_WORKSPACE: workspace missing, not 256-byte aligned or too small";
        case RK_ERR_DIMENSION: return "RK_ERR_DIMENSION: array extents do not agree";
        case RK_ERR_TOO_LARGE: return "RK_ERR_TOO_LARGE: an extent exceeds what the kernels can index";
        case RK_ERR_WAIT: return "RK_ERR_WAIT: a kernel gave up waiting for another workgroup (workspace not prepared, or shared by "
                                 "concurrent calls); the results of calls on it since the last check are invalid, prepare it again";
        default: break;
    }
    if (status > 0 && status < 10000) return hipGetErrorString((hipError_t)status);
    return "unknown rk status";
}

size_t rk_workspace_bytes(rk_opkind kind, rk_dtype dt, int ndim, const int64_t* shape, uint32_t dims_mask) {
    size_t need = WS_DESC_OFFSET;
    int64_t total = 0;
    if (kind == RK_KIND_ACCUMULATE && valid_dtype(dt) && valid_shape(ndim, shape, &total) && total > 0) {
        // descriptors of the look-back scan: one tagged word per 4 bytes of the value, per tile
        const Shape3 s = collapse3(ndim, shape, dims_mask);
        const size_t esz = dtype_size(dt) < 4 ? 4 : dtype_size(dt);
        const int64_t tile = (int64_t)scan_tile_waves(s.mid, esz) * WAVE * (16 / (int64_t)esz) * 8;      // the tile launch_scan picks
        const int64_t tpl = (s.mid + tile - 1) / tile, gpl = (tpl + WAVE - 1) / WAVE;
        // one tagged word per 4 bytes of the value per tile, one 128-byte line per group of 64 tiles
        // scans across rows publish 1 KiB of column totals per tile in the partials area: one flag each
        if (s.inner > 1) need += WS_PARTIALS_BYTES / 1024 * sizeof(uint64_t);
        if (s.inner == 1 && tpl > 1) need += ((size_t)(tpl * s.outer) * (esz / 4) + (size_t)(gpl * s.outer) * GROUP_DESC_STRIDE) * sizeof(uint64_t);
    }
    if (kind == RK_KIND_FINDALL && valid_shape(ndim, shape, &total) && total > 0) need += findall_workspace_need(total);
    return (need + 255) & ~(size_t)255;
}

int32_t rk_workspace_init(void* ws, size_t ws_bytes, void* stream) {
    if (ws == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (!is_aligned(ws, 256) || ws_bytes < WS_DESC_OFFSET) return RK_ERR_WORKSPACE;
    return workspace_init(ws, ws_bytes, (hipStream_t)stream);
}

int64_t rk_set_wait_budget(int64_t rounds) {
    const long long prev = wait_budget();
    g_wait_budget.store(rounds > 0 ? (long long)rounds : WAIT_BUDGET_DEFAULT, std::memory_order_relaxed);
    return (int64_t)prev;
}

int32_t rk_workspace_status(const void* ws, size_t ws_bytes, void* stream) {
    if (ws == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (!is_aligned(ws, 256) || ws_bytes < WS_DESC_OFFSET) return RK_ERR_WORKSPACE;
    uint32_t failed = 0;
    RK_HIP(hipMemcpyAsync(&failed, (const char*)ws + offsetof(WsHeader, wait_failed), sizeof(failed), hipMemcpyDeviceToHost, (hipStream_t)stream));
    RK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return failed != 0u ? RK_ERR_WAIT : RK_SUCCESS;
}

static int32_t mapreduce_dispatch(rk_map f, rk_op op, rk_dtype in, rk_dtype out, const void* A, int ndim, const int64_t* shape,
                                  uint32_t reduce_mask, void* R, const void* init, void* ws, size_t ws_bytes, void* stream,
                                  size_t partials_cap) {
    int64_t total = 0;
    if (!valid_dtype(in) || !valid_dtype(out)) return RK_ERR_INVALID_ARGUMENT;
    if ((int)f < RK_MAP_IDENTITY || (int)f > RK_MAP_ABS) return RK_ERR_INVALID_ARGUMENT;
    if ((int)op >= RK_OP_AND && (int)op <= RK_OP_XOR) return RK_ERR_UNSUPPORTED;       // bitwise operators: scans only
    if ((int)op < RK_OP_ADD || (int)op > RK_OP_MIN) return RK_ERR_INVALID_ARGUMENT;
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;                     // mapreduce.jl:91
    if (A == nullptr || R == nullptr) return RK_ERR_INVALID_ARGUMENT;
    reduce_mask &= (1u << ndim) - 1u;       // dims beyond ndim reduce nothing
    MapreduceArgs a{(int)f, (int)op, nullptr, A, ndim, shape, reduce_mask, R, init, ws, ws_bytes, (hipStream_t)stream, partials_cap};
    if (in == out) {
        switch (in) {
            case RK_F32: return mapreduce_f32(a);
            case RK_F16: return mapreduce_f16(a);
            case RK_F64: return mapreduce_f64(a);
            case RK_I32: return mapreduce_i32(a);
            case RK_I64: return mapreduce_i64(a);
            case RK_U8:  return mapreduce_u8(a);
            case RK_I8:  return mapreduce_i8(a);
            case RK_I16: return mapreduce_i16(a);
            case RK_U16: return mapreduce_u16(a);
            case RK_U32: return mapreduce_u32(a);
            case RK_U64: return mapreduce_u64(a);
            default: return RK_ERR_UNSUPPORTED;
        }
    }
    if (in == RK_I32 && out == RK_I64) return mapreduce_i32_i64(a);
    if (in == RK_U8 && (out == RK_I64 || out == RK_U64)) return mapreduce_u8_i64(a);   // sums of bytes: the same bits either way
    if (in == RK_U32 && out == RK_U64) return mapreduce_u32_u64(a);
    if (in == RK_I8 && out == RK_I64) return mapreduce_i8_i64(a);
    if (in == RK_I16 && out == RK_I64) return mapreduce_i16_i64(a);
    if (in == RK_U16 && out == RK_U64) return mapreduce_u16_u64(a);
    return RK_ERR_UNSUPPORTED;
}

int32_t rk_mapreduce(rk_map f, rk_op op, rk_dtype in, rk_dtype out, const void* A, int ndim, const int64_t* shape,
                     uint32_t reduce_mask, void* R, const void* init, void* ws, size_t ws_bytes, void* stream) {
    return mapreduce_dispatch(f, op, in, out, A, ndim, shape, reduce_mask, R, init, ws, ws_bytes, stream, WS_PARTIALS_BYTES);
}

// ---- wrapper arrays (transpose, PermutedDimsArray, reshape) in reductions and scans ---------------------------------------
// A permuted-dense array -- its strides are those of a dense column-major array with the dims in another order -- is
// a dense array once the dims are listed in memory order, and a reduction or scan over some of its dims is the same
// operation over the same dims of that dense array.  No kernel knows about strides: the entry points renumber the dims.
struct DenseOrder {
    int     order[RK_MAX_DIMS];      // order[k] = the logical dim that is k-th in memory (extents of 1 last)
    int64_t shape[RK_MAX_DIMS];      // extents in memory order
};
// false: the strides are not those of a permuted dense array (a view with gaps, a reversed or repeated dim)
static bool dense_order(int ndim, const int64_t* shape, const int64_t* strides, DenseOrder* o) {
    bool used[RK_MAX_DIMS] = {};
    int n = 0;
    int64_t expect = 1;
    for (;;) {
        int pick = -1;
        for (int d = 0; d < ndim; ++d)
            if (!used[d] && shape[d] != 1 && (strides ? strides[d] : expect) == expect && (strides || pick < 0)) { pick = d; break; }
        if (pick < 0) break;
        used[pick] = true;
        o->order[n] = pick;
        o->shape[n] = shape[pick];
        ++n;
        expect *= shape[pick];
    }
    for (int d = 0; d < ndim; ++d) {
        if (used[d]) continue;
        if (shape[d] != 1) return false;
        o->order[n] = d;
        o->shape[n] = 1;
        ++n;
    }
    return true;
}

int32_t rk_mapreduce_strided(rk_map f, rk_op op, rk_dtype in, rk_dtype out, const void* A, int ndim, const int64_t* shape,
                             const int64_t* a_strides, uint32_t reduce_mask, void* R, const int64_t* r_strides, const void* init,
                             void* ws, size_t ws_bytes, void* stream) {
    int64_t total = 0;
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    if (!valid_dtype(in) || !valid_dtype(out) || A == nullptr || R == nullptr) return RK_ERR_INVALID_ARGUMENT;
    reduce_mask &= (1u << ndim) - 1u;
    DenseOrder o{};
    if (!dense_order(ndim, shape, a_strides, &o)) return RK_ERR_UNSUPPORTED;
    uint32_t mask_mem = 0;
    for (int k = 0; k < ndim; ++k)
        if ((reduce_mask >> o.order[k]) & 1u) mask_mem |= 1u << k;
    // where the kernels put R: the kept dims in memory order, densely.  nat[d] = that stride of logical dim d
    int64_t nat[RK_MAX_DIMS] = {}, rshape[RK_MAX_DIMS], count = 1;
    for (int k = 0; k < ndim; ++k) {
        const int d = o.order[k];
        if ((reduce_mask >> d) & 1u) continue;
        nat[d] = count;
        count *= shape[d];
    }
    bool same = true;
    int64_t dense = 1;
    for (int d = 0; d < ndim; ++d) {
        const bool kept = !((reduce_mask >> d) & 1u);
        rshape[d] = kept ? shape[d] : 1;
        const int64_t want = r_strides ? r_strides[d] : dense;
        if (kept && shape[d] > 1 && want != nat[d]) same = false;
        dense *= rshape[d];
    }
    if (same) return mapreduce_dispatch(f, op, in, out, A, ndim, o.shape, mask_mem, R, init, ws, ws_bytes, stream, WS_PARTIALS_BYTES);
    // R is laid out otherwise (the transpose of mapreducedim!(identity, +, transpose(R), A)): reduce into the top of
    // the partials area, then one strided copy into R
    const size_t esz = dtype_size(out);
    const size_t temp_bytes = ((size_t)count * esz + 255) & ~(size_t)255;
    Workspace w{};
    if (temp_bytes > WS_PARTIALS_BYTES / 4) return RK_ERR_UNSUPPORTED;
    if (!carve_workspace(ws, ws_bytes, 0, &w)) return RK_ERR_WORKSPACE;
    void* temp = w.partials + WS_PARTIALS_BYTES - temp_bytes;
    const int32_t st = mapreduce_dispatch(f, op, in, out, A, ndim, o.shape, mask_mem, temp, init, ws, ws_bytes, stream,
                                          WS_PARTIALS_BYTES - temp_bytes);
    if (st != RK_SUCCESS) return st;
    rk_program prog{};
    prog.compute = (out == RK_F32 || out == RK_F16) ? RK_F32 : (out == RK_F64 ? RK_F64 : RK_I64);
    prog.n_operands = 1;
    prog.operands[0].ptr = temp;
    prog.operands[0].dtype = out;
    prog.operands[0].ndim = ndim;
    prog.operands[0].strided = 1;
    for (int d = 0; d < ndim; ++d) {
        prog.operands[0].shape[d] = rshape[d];
        prog.operands[0].strides[d] = rshape[d] > 1 ? nat[d] : 0;
    }
    prog.n_tokens = 1;
    prog.tokens[0] = 0;
    int64_t rs[RK_MAX_DIMS];
    dense = 1;
    for (int d = 0; d < ndim; ++d) {
        rs[d] = r_strides ? r_strides[d] : dense;
        dense *= rshape[d];
    }
    return rk_broadcast_strided(&prog, R, out, ndim, rshape, rs, stream);
}

int32_t rk_mapreduce_program(const rk_map_program* f, rk_op op, rk_dtype in, rk_dtype out, const void* A, int ndim,
                             const int64_t* shape, uint32_t reduce_mask, void* R, const void* init, void* ws, size_t ws_bytes,
                             void* stream) {
    int64_t total = 0;
    if (f == nullptr || !valid_dtype(in) || !valid_dtype(out)) return RK_ERR_INVALID_ARGUMENT;
    if ((int)op >= RK_OP_AND && (int)op <= RK_OP_XOR) return RK_ERR_UNSUPPORTED;       // bitwise operators: scans only
    if ((int)op < RK_OP_ADD || (int)op > RK_OP_MIN) return RK_ERR_INVALID_ARGUMENT;
    if (f->n_tokens < 1 || f->n_tokens > RK_MAP_MAX_TOKENS || f->n_consts < 0 || f->n_consts > RK_MAP_MAX_CONSTS) return RK_ERR_INVALID_ARGUMENT;
    const bool int_compute = in != RK_F32 && in != RK_F64;
    {   // operand 0 = the element, 1 .. n_consts = the constants; the value stack stays in registers
        const int32_t st = validate_tokens(f->tokens, f->n_tokens, 1 + f->n_consts, int_compute, INTERP_REG_DEPTH);
        if (st != RK_SUCCESS) return st;
        for (int i = 0; i < f->n_tokens; ++i)
            if (!token_basic(f->tokens[i])) return RK_ERR_UNSUPPORTED;      // pow, sin, cos, tanh: map first, then reduce
    }
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;                     // mapreduce.jl:91
    if (A == nullptr || R == nullptr) return RK_ERR_INVALID_ARGUMENT;
    reduce_mask &= (1u << ndim) - 1u;
    MapreduceArgs a{RK_MAP_PROGRAM, (int)op, f, A, ndim, shape, reduce_mask, R, init, ws, ws_bytes, (hipStream_t)stream};
    if (in == RK_F32 && out == RK_F32) return mapreduce_prog_f32(a);
    if (in == RK_F32 && out == RK_I64) return mapreduce_prog_f32_i64(a);
    if (in == RK_F64 && out == RK_F64) return mapreduce_prog_f64(a);
    if (in == RK_F64 && out == RK_I64) return mapreduce_prog_f64_i64(a);
    if (in == RK_I32 && out == RK_I32) return mapreduce_prog_i32(a);
    if (in == RK_I32 && out == RK_I64) return mapreduce_prog_i32_i64(a);
    if (in == RK_I64 && out == RK_I64) return mapreduce_prog_i64(a);
    if (in == RK_U8 && out == RK_I64) return mapreduce_prog_u8_i64(a);
    return RK_ERR_UNSUPPORTED;
}

int32_t rk_findminmax(int32_t want_max, rk_dtype in, const void* A, int ndim, const int64_t* shape, uint32_t reduce_mask,
                      void* vals, int64_t* cart_idx, void* ws, size_t ws_bytes, void* stream) {
    int64_t total = 0;
    if (!valid_dtype(in)) return RK_ERR_INVALID_ARGUMENT;
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    if (A == nullptr || (vals == nullptr && cart_idx == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    reduce_mask &= (1u << ndim) - 1u;
    FindArgs a{want_max ? 1 : 0, A, ndim, shape, reduce_mask, vals, cart_idx, ws, ws_bytes, (hipStream_t)stream};
    return findminmax_dispatch(in, a);
}

int32_t rk_findminmax_strided(int32_t want_max, rk_dtype in, const void* A, int ndim, const int64_t* shape, const int64_t* a_strides,
                              uint32_t reduce_mask, void* vals, int64_t* cart_idx, void* ws, size_t ws_bytes, void* stream) {
    int64_t total = 0;
    if (!valid_dtype(in)) return RK_ERR_INVALID_ARGUMENT;
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    if (A == nullptr || (vals == nullptr && cart_idx == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    reduce_mask &= (1u << ndim) - 1u;
    DenseOrder o{};
    if (!dense_order(ndim, shape, a_strides, &o)) return RK_ERR_UNSUPPORTED;
    // the kernels number the dims by their place in memory and lay the outputs out by the kept dims in that order; the
    // caller's outputs are dense in the LOGICAL order of the kept dims: served when the two orders agree (a transposed
    // matrix reduced along either dim, any wrapper reduced to one kept dim or to a scalar), declined otherwise
    // The same holds among the reduced dims: "the first of several equal winners" is the first in the wrapper's
    // column-major order, which is the order of the memory positions only when the reduced dims keep their order.
    uint32_t mask_mem = 0;
    int last_kept = -1, last_reduced = -1;
    for (int k = 0; k < ndim; ++k) {
        const int d = o.order[k];
        if (shape[d] == 1) { if ((reduce_mask >> d) & 1u) mask_mem |= 1u << k; continue; }
        if ((reduce_mask >> d) & 1u) {
            mask_mem |= 1u << k;
            if (d < last_reduced) return RK_ERR_UNSUPPORTED;
            last_reduced = d;
        } else {
            if (d < last_kept) return RK_ERR_UNSUPPORTED;
            last_kept = d;
        }
    }
    FindArgs a{want_max ? 1 : 0, A, ndim, o.shape, mask_mem, vals, cart_idx, ws, ws_bytes, (hipStream_t)stream};
    a.slot = o.order;        // memory dim k is the wrapper's dim order[k]: the index goes out in the wrapper's coordinates
    return findminmax_dispatch(in, a);
}


int32_t rk_accumulate(rk_op op, rk_dtype in, rk_dtype out, const void* in_ptr, void* out_ptr, int ndim, const int64_t* shape,
                      int dim, int32_t inclusive, const void* init, void* ws, size_t ws_bytes, void* stream) {
    int64_t total = 0;
    if (!valid_dtype(in) || !valid_dtype(out)) return RK_ERR_INVALID_ARGUMENT;
    if ((int)op < RK_OP_ADD || (int)op > RK_OP_XOR) return RK_ERR_INVALID_ARGUMENT;
    if (!valid_shape(ndim, shape, &total)) return RK_ERR_INVALID_ARGUMENT;
    if (dim < 1) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    if (in_ptr == nullptr || out_ptr == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (!inclusive && init == nullptr && (op == RK_OP_MAX || op == RK_OP_MIN)) return RK_ERR_INVALID_ARGUMENT;
    ScanArgs a{(int)op, in_ptr, out_ptr, ndim, shape, dim, inclusive, init, ws, ws_bytes, (hipStream_t)stream};
    if (in == out) {
        switch (in) {
            case RK_F32: return scan_f32(a);
            case RK_F64: return scan_f64(a);
            case RK_I32: return scan_i32(a);
            case RK_I64: return scan_i64(a);
            case RK_U32: return scan_u32(a);
            case RK_U64: return scan_u64(a);
            // 1- and 2-byte elements: scanned in 32 bits (Float16: in Float32, one rounding at the store), stored narrow
            case RK_I8:  return scan_i8(a);
            case RK_U8:  return scan_u8(a);
            case RK_I16: return scan_i16(a);
            case RK_U16: return scan_u16(a);
            case RK_F16: return scan_f16(a);
            default: return RK_ERR_UNSUPPORTED;
        }
    }
    if (in_ptr == out_ptr) return RK_ERR_INVALID_ARGUMENT;   // aliasing needs equal element sizes
    if (in == RK_U8 && out == RK_I64) return scan_u8_i64(a);
    if (in == RK_U8 && out == RK_I32) return scan_u8_i32(a);
    return RK_ERR_UNSUPPORTED;
}

int32_t rk_accumulate_strided(rk_op op, rk_dtype in, rk_dtype out, const void* in_ptr, void* out_ptr, int ndim, const int64_t* shape,
                              const int64_t* in_strides, const int64_t* out_strides, int dim, int32_t inclusive, const void* init,
                              void* ws, size_t ws_bytes, void* stream) {
    int64_t total = 0;
    if (!valid_shape(ndim, shape, &total) || dim < 1) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    DenseOrder oi{}, oo{};
    if (!dense_order(ndim, shape, in_strides, &oi) || !dense_order(ndim, shape, out_strides, &oo)) return RK_ERR_UNSUPPORTED;
    for (int k = 0; k < ndim; ++k)
        if (oi.order[k] != oo.order[k]) return RK_ERR_UNSUPPORTED;     // input and output must be laid out alike
    int dim_mem = dim;                                                 // dim > ndim: a copy, whatever the layout
    for (int k = 0; k < ndim; ++k)
        if (oi.order[k] == dim - 1) dim_mem = k + 1;
    return rk_accumulate(op, in, out, in_ptr, out_ptr, ndim, oi.shape, dim_mem, inclusive, init, ws, ws_bytes, stream);
}

int32_t rk_accumulate_static(rk_op op, rk_dtype in, rk_dtype out, const void* in_ptr, void* out_ptr, int ndim, const int64_t* shape,
                             int dim, int32_t inclusive, const void* init, void* stream) {
    // size check first: it needs no device, and a request that cannot be served must not prepare anything
    int64_t total = 0;
    if (!valid_dtype(in) || !valid_dtype(out) || !valid_shape(ndim, shape, &total) || dim < 1) return RK_ERR_INVALID_ARGUMENT;
    if (total == 0) return RK_SUCCESS;
    const uint32_t mask = dim <= ndim ? (1u << (dim - 1)) : 0u;
    if (rk_workspace_bytes(RK_KIND_ACCUMULATE, out, ndim, shape, mask) > RK_STATIC_SCRATCH_BYTES) return RK_ERR_TOO_LARGE;
    if (in_ptr == nullptr || out_ptr == nullptr) return RK_ERR_INVALID_ARGUMENT;
    void* ws = nullptr;
    const int32_t st = static_scratch((hipStream_t)stream, &ws);
    if (st != RK_SUCCESS) return st;
    return rk_accumulate(op, in, out, in_ptr, out_ptr, ndim, shape, dim, inclusive, init, ws, RK_STATIC_SCRATCH_BYTES, stream);
}

int32_t rk_accumulate_static_status(void* stream) {
    int dev = 0;
    RK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return RK_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    void* ptr = g_static_ptr[dev];
    if (ptr == nullptr) return RK_SUCCESS;                 // never used on this device
    const int32_t st = rk_workspace_status(ptr, RK_STATIC_SCRATCH_BYTES, stream);
    if (st == RK_ERR_WAIT) {                               // reported once; the array starts afresh
        const int32_t again = workspace_init(ptr, RK_STATIC_SCRATCH_BYTES, (hipStream_t)stream);
        if (again != RK_SUCCESS) return again;
        RK_HIP(hipStreamSynchronize((hipStream_t)stream));
    }
    return st;
}

}  // extern "C"
