// C ABI of the gfx950 backend (see include/ferrum_hip.h): objects, validation
// and kernel selection.  Argument checks mirror the reference's operator
// methods (src/ops/transformer.rs:96-297, src/ops/mod.rs:23-609) and its
// binding checks (src/metal/mod.rs:840-897): shapes, ownership, bounds,
// alignment and input/output aliasing are rejected before anything launches.
#include <cmath>
#include <cstdarg>
#include <mutex>
#include <cstring>
#include <new>
#include <vector>

#include "internal.hpp"

namespace fh {

static thread_local std::string g_last_error;

fh_status fail(fh_status code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

fh_status hip_fail(hipError_t err, const char* what) {
    fh_status code = err == hipErrorOutOfMemory ? FH_ERR_ALLOCATION : FH_ERR_DISPATCH;
    return fail(code, "%s: %s", what, hipGetErrorString(err));
}

namespace {

#define FH_HIP(expr)                                        \
    do {                                                    \
        hipError_t _e = (expr);                             \
        if (_e != hipSuccess) return hip_fail(_e, #expr);   \
    } while (0)

struct Range {
    const uint8_t* begin;
    size_t bytes;
};

bool overlaps(const Range& a, const Range& b) {
    return a.begin < b.begin + b.bytes && b.begin < a.begin + a.bytes;
}

// Resolves a view to a device pointer after ownership, bounds and alignment
// checks.  `elements` is the number of dtype-sized elements the op touches.
fh_status resolve(const fh_device* device, const fh_view* view, uint64_t elements, const char* what,
                  Range* out, size_t alignment = 16) {
    if (view == nullptr || view->buffer == nullptr)
        return fail(FH_ERR_RANGE, "%s: null view", what);
    if (view->dtype > FH_BF16) return fail(FH_ERR_DTYPE, "%s: unknown dtype %u", what, view->dtype);
    if (view->buffer->device != device) {
        g_last_error = std::string(what) + ": buffer belongs to another device";
        return FH_ERR_DEVICE_MISMATCH;
    }
    uint64_t bytes = elements * dtype_bytes(view->dtype);
    if (view->offset > view->buffer->bytes || bytes > view->buffer->bytes - view->offset)
        return fail(FH_ERR_RANGE, "%s: view [%zu, +%llu) exceeds buffer of %zu bytes", what,
                    view->offset, (unsigned long long)bytes, view->buffer->bytes);
    if (view->offset % alignment != 0)
        return fail(FH_ERR_RANGE, "%s: offset %zu is not %zu-byte aligned", what, view->offset,
                    alignment);
    out->begin = static_cast<const uint8_t*>(view->buffer->ptr) + view->offset;
    out->bytes = (size_t)bytes;
    return FH_OK;
}

bool fits_u32(uint64_t v) { return v <= 0xffffffffull; }

// Device scratch: kCounterWords zeroed counter words followed by a data area
// of at least `data_bytes`.  Growing it waits for the stream first.  Recorded executions
// carry the scratch address in their kernel arguments, so a block that is outgrown while
// any of them is alive is kept (they replay on it unchanged) and freed with the last one.
fh_status ensure_scratch(fh_device* d, size_t data_bytes) {
    const size_t counter_bytes = fh_device::kCounterWords * sizeof(uint32_t);
    if (d->scratch != nullptr && d->scratch_bytes >= counter_bytes + data_bytes) return FH_OK;
    if (d->capturing)
        return fail(FH_ERR_SYNCHRONIZATION, "device scratch must grow: run the operator once before recording it");
    FH_HIP(hipStreamSynchronize(d->stream));
    // at least twice the old data area, so the blocks kept for recordings add up to less than the live one
    const size_t old_data = d->scratch_bytes > counter_bytes ? d->scratch_bytes - counter_bytes : 0;
    if (data_bytes < 2 * old_data) data_bytes = 2 * old_data;
    if (d->scratch) {
        if (d->live_graphs > 0) {
            d->retired_scratch.push_back(d->scratch);
        } else {
            (void)hipFree(d->scratch);
        }
    }
    d->scratch = nullptr;
    d->scratch_bytes = 0;
    size_t cap = counter_bytes + (data_bytes < (16u << 20) ? (16u << 20) : data_bytes);
    hipError_t e = hipMalloc(&d->scratch, cap);
    if (e != hipSuccess) return fail(FH_ERR_ALLOCATION, "hipMalloc(%zu): %s", cap, hipGetErrorString(e));
    d->scratch_bytes = cap;
    FH_HIP(hipMemsetAsync(d->scratch, 0, counter_bytes, d->stream));
    return FH_OK;
}
// A block the library owns for its own temporaries (it holds no count on the device), grown like
// the scratch: outside recordings only, by at least 2x, old blocks kept for the recorded executions
// that carry their address.
fh_status ensure_block(fh_device* d, fh_buffer*& slot, size_t bytes, const char* what) {
    if (slot != nullptr && slot->bytes >= bytes) return FH_OK;
    if (d->capturing)
        return fail(FH_ERR_SYNCHRONIZATION, "%s must grow: run the call once before recording it", what);
    FH_HIP(hipStreamSynchronize(d->stream));
    if (slot == nullptr) {
        slot = new (std::nothrow) fh_buffer();
        if (slot == nullptr) return fail(FH_ERR_ALLOCATION, "out of host memory");
        slot->device = d;
    }
    if (bytes < 2 * slot->bytes) bytes = 2 * slot->bytes;
    if (slot->ptr) {
        if (d->live_graphs > 0) d->retired_scratch.push_back(slot->ptr);
        else (void)hipFree(slot->ptr);
    }
    slot->ptr = nullptr;
    slot->bytes = 0;
    hipError_t e = hipMalloc(&slot->ptr, bytes);
    if (e != hipSuccess) return fail(FH_ERR_ALLOCATION, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
    slot->bytes = bytes;
    return FH_OK;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// ---- matrices whose rows are stored padded (Q8_0 rows of 32 n weights, n not a multiple of 8) ----
// An entry point that meets one runs on the matrix as it is stored (rows of stored_cols weights,
// the added blocks empty) and on its activations rewritten to that width, zeros in the added
// columns, in a block of the device's own.  Everything behind that point is the ordinary path.
fh_qmatrix as_stored(const fh_qmatrix* w) {
    fh_qmatrix m = *w;
    m.cols = w->stored_cols;
    return m;
}

struct PaddedActivations {
    struct Item {
        const fh_view* x;
        uint64_t pieces;   // rows x parts: runs of `cols` elements
        const char* what;
        fh_view* out;
        Range range;
    };
    fh_device* device;
    uint64_t cols, stored;
    Item items[2];
    int count = 0;
    PaddedActivations(fh_device* d, const fh_qmatrix* w) : device(d), cols(w->cols), stored(w->stored_cols) {}
    void add(const fh_view* x, uint64_t pieces, const char* what, fh_view* out) {
        items[count++] = Item{x, pieces, what, out, Range{nullptr, 0}};
    }
    // checks the views, then writes the padded copies and points `out` at them
    fh_status run() {
        size_t at = 0, offsets[2] = {0, 0};
        for (int i = 0; i < count; ++i) {
            Item& it = items[i];
            if (!fits_u32(it.pieces * stored)) return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
            fh_status st = resolve(device, it.x, it.pieces * cols, it.what, &it.range);
            if (st != FH_OK) return st;
            offsets[i] = at;
            at += align256((size_t)(it.pieces * stored) * dtype_bytes(it.x->dtype));
        }
        fh_status st = ensure_block(device, device->padded_rows, at, "the block for padded activations");
        if (st != FH_OK) return st;
        for (int i = 0; i < count; ++i) {
            const Item& it = items[i];
            launch_pad_rows(device->stream, it.range.begin, static_cast<uint8_t*>(device->padded_rows->ptr) + offsets[i],
                            (size_t)it.pieces, (size_t)cols, (size_t)stored, dtype_bytes(it.x->dtype));
            *it.out = fh_view{device->padded_rows, offsets[i], it.x->dtype};
        }
        FH_HIP(hipGetLastError());
        return FH_OK;
    }
    // an output may not alias the activations as the caller passed them
    fh_status keep_apart(const fh_view* y, uint64_t elements, const char* what, const char* message) const {
        Range yr;
        fh_status st = resolve(device, y, elements, what, &yr);
        if (st != FH_OK) return st;
        for (int i = 0; i < count; ++i)
            if (overlaps(items[i].range, yr)) return fail(FH_ERR_RANGE, "%s", message);
        return FH_OK;
    }
};

uint32_t* scratch_counters(fh_device* d) { return static_cast<uint32_t*>(d->scratch); }
uint8_t* scratch_data(fh_device* d) {
    return static_cast<uint8_t*>(d->scratch) + fh_device::kCounterWords * sizeof(uint32_t);
}

// Points a GEMV launch that cuts K into segments at the device scratch
// (partial sums and one zeroed counter word per row tile and batch row).
fh_status prepare_gemv(fh_device* d, GemvArgs& a) {
    const GemvScratch plan = gemv_scratch(a);
    if (plan.segments > 1) {
        if ((uint64_t)plan.tiles * a.m > fh_device::kCounterWords)
            return fail(FH_ERR_SHAPE, "projection needs %llu row tiles, more than the K-split scratch holds",
                        (unsigned long long)plan.tiles * a.m);
        fh_status st = ensure_scratch(d, (size_t)plan.segments * a.m * a.n * sizeof(float));
        if (st != FH_OK) return st;
        a.partials = reinterpret_cast<float*>(scratch_data(d));
        a.counters = scratch_counters(d);
    }
    return FH_OK;
}

// Runs a GEMV launch of any batch size: the batch is cut into runs that fit the grid's z
// extent and, where K is cut into segments, the counter words (one per row tile and batch
// entry).  A launch that carries a shared expert is not cut.
fh_status run_gemv(fh_device* d, GemvArgs a, const char** name) {
    const GemvScratch plan = gemv_scratch(a);
    uint64_t most = 65535u;
    if (plan.segments > 1 && plan.tiles > 0) most = std::min<uint64_t>(most, fh_device::kCounterWords / plan.tiles);
    if (a.x_mode == kXDivide && a.x_div > 1) most -= most % a.x_div;   // the routes of a token stay together
    if (a.m <= most || a.shared_w != nullptr || most == 0) {
        fh_status st = prepare_gemv(d, a);
        if (st != FH_OK) return st;
        if (a.m > 65535u) return fail(FH_ERR_SHAPE, "batch of %u entries exceeds the launch grid", a.m);
        *name = launch_gemv(d->stream, a);
        return FH_OK;
    }
    const uint32_t total = a.m;
    const size_t x_row = (size_t)a.k * dtype_bytes(a.x_dtype) * (a.x_mode == kXSiluMul ? 2 : 1);
    const size_t y_row = (size_t)a.n * dtype_bytes(a.y_dtype);
    const uint32_t stride = a.meta_stride == 0 ? 3u : a.meta_stride;
    for (uint32_t first = 0; first < total; first += (uint32_t)most) {
        GemvArgs part = a;
        part.m = std::min<uint32_t>((uint32_t)most, total - first);
        part.y = static_cast<uint8_t*>(a.y) + first * y_row;
        if (a.metadata != nullptr) part.metadata = a.metadata + (size_t)first * stride;
        if (a.x_mode == kXPlain || a.x_mode == kXSiluMul) {
            part.x = static_cast<const uint8_t*>(a.x) + first * x_row;
            part.x_rows = part.m;
        } else if (a.x_mode == kXDivide) {
            const uint32_t div = a.x_div == 0 ? 1u : a.x_div;
            part.x = static_cast<const uint8_t*>(a.x) + (size_t)(first / div) * x_row;
            part.x_rows = part.m / div;
        }   // kXGather reads the token row named by each entry's metadata: x stays whole
        fh_status st = prepare_gemv(d, part);
        if (st != FH_OK) return st;
        *name = launch_gemv(d->stream, part);
    }
    return FH_OK;
}

// Frees device memory now, or after the recording in progress has ended.
void release_memory(fh_device* d, void* ptr) {
    if (ptr == nullptr) return;
    if (d != nullptr && d->closed) {
        (void)hipFree(ptr);   // synchronizes by itself; the stream no longer exists
        return;
    }
    if (d != nullptr && d->capturing) {
        d->deferred_frees.push_back(ptr);
        return;
    }
    if (d != nullptr) (void)hipStreamSynchronize(d->stream);
    (void)hipFree(ptr);
}

// One object created on the device is gone (or the caller's handle is); the last one frees it.
void drop_device_handle(fh_device* d) {
    if (d != nullptr && --d->handles == 0) delete d;
}

void drain_deferred(fh_device* d) {
    if (d->deferred_frees.empty() && d->deferred_graphs.empty()) return;
    (void)hipStreamSynchronize(d->stream);
    for (void* ptr : d->deferred_frees) (void)hipFree(ptr);
    for (auto& g : d->deferred_graphs) {
        (void)hipGraphExecDestroy(g.first);
        (void)hipGraphDestroy(g.second);
    }
    d->deferred_frees.clear();
    d->deferred_graphs.clear();
}

int64_t tuning(const fh_device* d, const char* key) {
    auto it = d->tuning.find(key);
    return it == d->tuning.end() ? 0 : it->second;
}

}  // namespace
}  // namespace fh

using namespace fh;

// Scratch of the entry point that allocates nothing: the K-segment partial sums and the
// row-tile counters of the GEMV.  Every device the library runs on holds its own copy of
// the array at its own address for the life of the process; `scratch` itself is only the
// host-side name of the symbol, the device address comes from hipGetSymbolAddress.
constexpr size_t kFixedCounterWords = 4096;
constexpr size_t kFixedScratchBytes = 1u << 20;   // 16 KiB of counters, then partial sums
static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];

static_assert(kXDivide > FH_INPUT_SILU_MUL, "the row-divide mode is internal: it has no public input form");
static_assert(kXPlain == FH_INPUT_ROWS && kXGather == FH_INPUT_GATHER && kXSiluMul == FH_INPUT_SILU_MUL,
              "the kernel's input modes are the ABI's input forms");

extern "C" {

const char* fh_last_error(void) { return g_last_error.c_str(); }

fh_status fh_device_create(int32_t ordinal, fh_device** out) {
    if (out == nullptr) return fail(FH_ERR_PARAMETER, "fh_device_create: null output");
    *out = nullptr;
    int count = 0;
    FH_HIP(hipGetDeviceCount(&count));
    if (ordinal < 0 || ordinal >= count)
        return fail(FH_ERR_DISPATCH, "no HIP device %d (found %d)", ordinal, count);
    FH_HIP(hipSetDevice(ordinal));
    fh_device* d = new (std::nothrow) fh_device();
    if (d == nullptr) return fail(FH_ERR_ALLOCATION, "out of host memory");
    d->ordinal = ordinal;
    hipError_t e = hipGetDeviceProperties(&d->props, ordinal);
    if (e != hipSuccess) {
        delete d;
        return hip_fail(e, "hipGetDeviceProperties");
    }
    if (std::strncmp(d->props.gcnArchName, "gfx950", 6) != 0) {
        fh_status st = fail(FH_ERR_DISPATCH, "kernels are built for gfx950 only; device %d is %s",
                            ordinal, d->props.gcnArchName);
        delete d;
        return st;
    }
    e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete d;
        return hip_fail(e, "hipStreamCreateWithFlags");
    }
    d->tuning["k_quant_gemv_ksplit"] = 0;   // 0 = automatic
    d->tuning["gemm_min_rows"] = 2;         // smallest M that takes the MFMA tile path
    d->tuning["gemm_wide_shape"] = 1;       // matrix instruction of the 128- and 256-row tiles: 0 = 16x16x32, 1 = whichever is estimated faster, 2 = 32x32x16
    d->tuning["gemm_wide32_tile"] = 0;      // 0 = by shape; 12, 14, 15 (128-row tile x 64, 128, 160 columns), 24, 25 (256-row tile)
    d->tuning["gemm_wide_min_rows"] = 33;   // smallest M that takes the 256-row tile (it wins from there up)
    d->tuning["gemm_skinny_max_rows"] = 64; // largest M that takes the register-dequant MFMA kernel (0 = never)
    d->tuning["expert_grouped_min_assignments"] = 32;  // fewest assignments grouped by expert (0 = never)
    d->tuning["moe_fold_route"] = 1;        // fh_moe_ffn, one token: the gate|up launch routes the token itself (0 = a moe_route launch first)
    d->tuning["gemm_few_tiles_split"] = 1;  // up to 16 rows and few weight tiles per workgroup: super-blocks dealt over the waves (0 = whole tiles per wave)
    d->tuning["moe_fold_combine"] = 1;      // fh_moe_ffn with few tokens: down projection and weighted sum in one launch (0 = two)
    d->tuning["gemm_resident"] = 1;         // rows that fit LDS whole take the rows-resident kernel (0 = square tiles)
    d->tuning["gemv_stream_own_loads"] = 1; // the streamed Q4_K GEMV's waves load the super-blocks they multiply (tiles of up to 14 rows); 0: the tile row by row
    d->tuning["expert_weight_ring"] = 1;    // grouped Q4_K / Q6_K expert projection with short rows: weights through LDS rings (0 = straight into registers)
    d->tuning["gemv_stream"] = 1;           // dense Q4_K / Q6_K GEMV on the streamed matrix-core kernel: 0 never, 1 where it wins, 2 wherever it runs
    d->tuning["moe_routing_temporary_limit"] = 128ll << 20;  // bytes of routing temporaries per SparseMoe chunk (src/metal/legacy.rs:95)
    d->tuning["gemm_f32_min_rows"] = 0;     // f32 activations take the f16 tile kernels from this many rows (0 = never)
    d->tuning["probe_read_form"] = 0;       // fh_probe_read: 100 x threads per workgroup + loads per lane (+ 1000000: LDS-direct loads); 0 = 256 x 8
    fh_status st = ensure_scratch(d, 0);
    if (st == FH_OK) {
        // This device's address of the fixed scratch (the device is current).  Its counters are set to zero
        // once per GPU and process: launches leave them at zero, and a second handle on a GPU whose first
        // handle has a K-split launch in flight must not reset that launch's tickets.
        void* fixed = nullptr;
        e = hipGetSymbolAddress(&fixed, HIP_SYMBOL(scratch));
        if (e == hipSuccess) {
            static std::mutex zero_lock;
            static bool zeroed[256] = {};
            std::lock_guard<std::mutex> hold(zero_lock);
            if (ordinal < 256 && !zeroed[ordinal]) {
                e = hipMemsetAsync(fixed, 0, kFixedCounterWords * sizeof(uint32_t), d->stream);
                if (e == hipSuccess) e = hipStreamSynchronize(d->stream);
                if (e == hipSuccess) zeroed[ordinal] = true;
            }
        }
        if (e != hipSuccess) st = hip_fail(e, "fixed scratch");
        d->fixed_scratch = fixed;
    }
    if (st != FH_OK) {
        if (d->scratch) (void)hipFree(d->scratch);
        (void)hipStreamDestroy(d->stream);
        delete d;
        return st;
    }
    *out = d;
    return FH_OK;
}

void fh_device_destroy(fh_device* device) {
    if (device == nullptr) return;
    (void)hipSetDevice(device->ordinal);
    if (device->closed) return;
    // what was put off during a recording goes first, while the stream it waits on exists
    if (device->capturing) {
        hipGraph_t abandoned = nullptr;
        (void)hipStreamEndCapture(device->stream, &abandoned);
        if (abandoned) (void)hipGraphDestroy(abandoned);
        device->capturing = false;
    }
    drain_deferred(device);
    if (device->stream) {
        (void)hipStreamSynchronize(device->stream);
        (void)hipStreamDestroy(device->stream);
        device->stream = nullptr;
    }
    if (device->scratch) (void)hipFree(device->scratch);
    if (device->workspace) {
        if (device->workspace->ptr) (void)hipFree(device->workspace->ptr);
        delete device->workspace;
        device->workspace = nullptr;
    }
    if (device->padded_rows) {
        if (device->padded_rows->ptr) (void)hipFree(device->padded_rows->ptr);
        delete device->padded_rows;
        device->padded_rows = nullptr;
    }
    for (void* old : device->retired_scratch) (void)hipFree(old);
    device->retired_scratch.clear();
    device->scratch = nullptr;
    device->scratch_bytes = 0;
    device->closed = true;
    drop_device_handle(device);
}

fh_status fh_device_properties(const fh_device* device, fh_device_props* out) {
    if (device == nullptr || out == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", device->props.name);
    if (out->name[0] == '\0')   // some driver stacks leave the marketing name empty
        std::snprintf(out->name, sizeof(out->name), "%.40s, %d CUs, %.0f GiB", device->props.gcnArchName,
                      device->props.multiProcessorCount, (double)device->props.totalGlobalMem / (1 << 30));
    std::snprintf(out->arch, sizeof(out->arch), "%s", device->props.gcnArchName);
    out->compute_units = device->props.multiProcessorCount;
    out->wavefront = device->props.warpSize;
    out->clock_khz = device->props.clockRate;
    out->memory_clock_khz = device->props.memoryClockRate;
    out->memory_bus_bits = device->props.memoryBusWidth;
    out->lds_bytes_per_block = (int32_t)device->props.sharedMemPerBlock;
    out->global_bytes = device->props.totalGlobalMem;
    out->l2_bytes = (uint64_t)device->props.l2CacheSize;
    return FH_OK;
}

fh_status fh_synchronize(fh_device* device) {
    if (device && device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null device");
    hipError_t e = hipStreamSynchronize(device->stream);
    if (e != hipSuccess) return fail(FH_ERR_SYNCHRONIZATION, "stream: %s", hipGetErrorString(e));
    return FH_OK;
}

const char* fh_last_operation(const fh_device* device) {
    return device ? device->last_operation : "";
}

void* fh_device_stream(fh_device* device) { return device ? device->stream : nullptr; }

fh_status fh_set_tuning(fh_device* device, const char* key, int64_t value) {
    if (device == nullptr || key == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    auto it = device->tuning.find(key);
    if (it == device->tuning.end()) return fail(FH_ERR_PARAMETER, "unknown tuning key %s", key);
    std::string k(key);
    bool ok = true;
    if (k == "k_quant_gemv_ksplit") {
        // set_k_quant_gemv_ksplit: 0 or a power of two up to 8
        ok = value == 0 || value == 1 || value == 2 || value == 4 || value == 8;
    } else if (k == "gemm_min_rows") {
        ok = value >= 2;
    } else if (k == "gemm_resident" || k == "moe_fold_combine" || k == "moe_fold_route") {
        ok = value == 0 || value == 1;
    } else if (k == "gemm_few_tiles_split" || k == "gemv_stream_own_loads" || k == "expert_weight_ring") {
        ok = value == 0 || value == 1;
    } else if (k == "gemv_stream") {
        ok = value >= 0 && value <= 2;
    } else if (k == "gemm_wide_shape") {
        ok = value >= 0 && value <= 2;
    } else if (k == "gemm_wide32_tile") {
        ok = value == 0 || value == 12 || value == 13 || value == 14 || value == 15 || value == 24 || value == 25;
    } else if (k == "gemm_wide_min_rows") {
        ok = value >= 1;
    } else if (k == "gemm_skinny_max_rows") {
        ok = value >= 0 && value <= 64;
    } else if (k == "expert_grouped_min_assignments") {
        ok = value >= 0;
    } else if (k == "gemm_f32_min_rows") {
        ok = value == 0 || value >= 2;
    } else if (k == "probe_read_form") {
        ok = value == 0 || value == 25604 || value == 25608 || value == 25616 || value == 51204 || value == 51208 ||
             value == 102404 || value == 102408 || value == 1025608 || value == 1025616 || value == 1051208;
    } else if (k == "moe_routing_temporary_limit") {
        // set_moe_routing_temporary_limit (src/metal/legacy.rs:523-531): positive, on an idle device
        ok = value > 0 && !device->capturing;
    }
    if (!ok) return fail(FH_ERR_PARAMETER, "value %lld is out of range for %s", (long long)value, key);
    it->second = value;
    return FH_OK;
}

fh_status fh_get_tuning(const fh_device* device, const char* key, int64_t* value) {
    if (device == nullptr || key == nullptr || value == nullptr)
        return fail(FH_ERR_PARAMETER, "null argument");
    auto it = device->tuning.find(key);
    if (it == device->tuning.end()) return fail(FH_ERR_PARAMETER, "unknown tuning key %s", key);
    *value = it->second;
    return FH_OK;
}

// ---- buffers -------------------------------------------------------------------

fh_status fh_buffer_alloc(fh_device* device, size_t bytes, fh_buffer** out) {
    if (device && device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (device == nullptr || out == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    *out = nullptr;
    if (bytes == 0) return fail(FH_ERR_ALLOCATION, "zero-length buffer");
    FH_HIP(hipSetDevice(device->ordinal));
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return fail(FH_ERR_ALLOCATION, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
    e = hipMemsetAsync(p, 0, bytes, device->stream);
    if (e != hipSuccess) {
        (void)hipFree(p);
        return hip_fail(e, "hipMemsetAsync");
    }
    fh_buffer* b = new (std::nothrow) fh_buffer();
    if (b == nullptr) {
        (void)hipFree(p);
        return fail(FH_ERR_ALLOCATION, "out of host memory");
    }
    b->device = device;
    ++device->handles;
    b->ptr = p;
    b->bytes = bytes;
    *out = b;
    return FH_OK;
}

void fh_buffer_free(fh_buffer* buffer) {
    if (buffer == nullptr) return;
    release_memory(buffer->device, buffer->ptr);
    drop_device_handle(buffer->device);
    delete buffer;
}

size_t fh_buffer_size(const fh_buffer* buffer) { return buffer ? buffer->bytes : 0; }
void* fh_buffer_device_ptr(fh_buffer* buffer) { return buffer ? buffer->ptr : nullptr; }

fh_status fh_buffer_upload(fh_buffer* buffer, size_t offset, const void* src, size_t bytes) {
    if (buffer && buffer->device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (buffer == nullptr || (src == nullptr && bytes)) return fail(FH_ERR_PARAMETER, "null argument");
    if (buffer->device->closed) return fail(FH_ERR_DEVICE_MISMATCH, "the buffer's device has been destroyed");
    if (offset > buffer->bytes || bytes > buffer->bytes - offset)
        return fail(FH_ERR_RANGE, "upload [%zu, +%zu) exceeds buffer of %zu bytes", offset, bytes,
                    buffer->bytes);
    if (bytes == 0) return FH_OK;
    hipStream_t s = buffer->device->stream;
    FH_HIP(hipMemcpyAsync(static_cast<uint8_t*>(buffer->ptr) + offset, src, bytes,
                          hipMemcpyHostToDevice, s));
    FH_HIP(hipStreamSynchronize(s));
    return FH_OK;
}

fh_status fh_buffer_download(const fh_buffer* buffer, size_t offset, void* dst, size_t bytes) {
    if (buffer && buffer->device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (buffer == nullptr || (dst == nullptr && bytes)) return fail(FH_ERR_PARAMETER, "null argument");
    if (buffer->device->closed) return fail(FH_ERR_DEVICE_MISMATCH, "the buffer's device has been destroyed");
    if (offset > buffer->bytes || bytes > buffer->bytes - offset)
        return fail(FH_ERR_RANGE, "download [%zu, +%zu) exceeds buffer of %zu bytes", offset, bytes,
                    buffer->bytes);
    if (bytes == 0) return FH_OK;
    hipStream_t s = buffer->device->stream;
    hipError_t e = hipMemcpyAsync(dst, static_cast<const uint8_t*>(buffer->ptr) + offset, bytes,
                                  hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpyAsync");
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail(FH_ERR_SYNCHRONIZATION, "stream: %s", hipGetErrorString(e));
    return FH_OK;
}

fh_status fh_buffer_fill_zero(fh_buffer* buffer, size_t offset, size_t bytes) {
    if (buffer && buffer->device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (buffer == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (offset > buffer->bytes || bytes > buffer->bytes - offset)
        return fail(FH_ERR_RANGE, "fill exceeds buffer");
    if (bytes == 0) return FH_OK;
    FH_HIP(hipMemsetAsync(static_cast<uint8_t*>(buffer->ptr) + offset, 0, bytes,
                          buffer->device->stream));
    return FH_OK;
}

// ---- packed weights --------------------------------------------------------------

static bool f16_finite(const uint8_t* p) { return ((p[1] >> 2) & 0x1f) != 0x1f; }

fh_status fh_qmatrix_create(fh_device* device, uint32_t ggml_type, uint64_t rows, uint64_t cols,
                            uint64_t experts, const void* packed, size_t packed_len,
                            fh_qmatrix** out) {
    if (device && device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (device == nullptr || out == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    *out = nullptr;
    const size_t bb = block_bytes(ggml_type);
    if (bb == 0) return fail(FH_ERR_GGUF, "unsupported quantized weight type %u", ggml_type);
    const char* name = ggml_type == kQ4K   ? "Q4_K"
                       : ggml_type == kQ5K ? "Q5_K"
                       : ggml_type == kQ6K ? "Q6_K"
                       : ggml_type == kQ8_0 ? "Q8_0"
                                            : "IQ4_XS";
    // a row is whole blocks: super-blocks of 256 weights, or for Q8_0 the 32-weight blocks of its GGML
    // geometry (src/loader/gguf.rs:99)
    const uint64_t unit = ggml_type == kQ8_0 ? 32 : 256;
    const size_t unit_bytes = ggml_type == kQ8_0 ? 34 : bb;
    if (rows == 0 || cols == 0 || cols % unit != 0)
        return fail(FH_ERR_SHAPE, "%s matrix requires nonempty rows and columns divisible by block size %u",
                    name, (unsigned)unit);
    if (experts == 0) return fail(FH_ERR_SHAPE, "quantized expert matrix row geometry mismatch");
    const uint64_t stored_cols = (cols + 255) / 256 * 256;
    unsigned __int128 total_rows = (unsigned __int128)rows * experts;
    unsigned __int128 byte_len = total_rows * (cols / unit) * unit_bytes;
    unsigned __int128 stored_len = total_rows * (stored_cols / 256) * bb;
    if (total_rows > 0xffffffffull || stored_len > (unsigned __int128)SIZE_MAX / 2)
        return fail(FH_ERR_SHAPE, "packed matrix byte size overflow");
    if (packed == nullptr) return fail(FH_ERR_PARAMETER, "null payload");
    if (packed_len % unit_bytes != 0)
        return fail(FH_ERR_GGUF, "tensor %s stream ended inside a block", name);
    if ((unsigned __int128)packed_len != byte_len)
        return fail(FH_ERR_SHAPE, "%s payload is %zu bytes, geometry needs %llu", name, packed_len,
                    (unsigned long long)byte_len);
    const uint8_t* p = static_cast<const uint8_t*>(packed);
    for (size_t off = 0; off < packed_len; off += unit_bytes) {
        bool ok = ggml_type == kQ6K     ? f16_finite(p + off + 208)
                  : ggml_type == kIQ4XS || ggml_type == kQ8_0 ? f16_finite(p + off)
                                        : (f16_finite(p + off) && f16_finite(p + off + 2));
        if (!ok) return fail(FH_ERR_WEIGHT, "%s scale must be finite", name);
    }
    // Q8_0 rows that do not end on a run of eight blocks are stored with the run completed by
    // empty blocks (scale and quants zero): the kernels then see rows of `stored_cols` weights,
    // and the entry points bring the activations to that width (pad_activations below)
    std::vector<uint8_t> staged;
    const size_t upload_len = (size_t)stored_len;
    if (stored_cols != cols) {
        try {
            staged.assign(upload_len, 0);
        } catch (const std::bad_alloc&) {
            return fail(FH_ERR_ALLOCATION, "out of host memory");
        }
        const size_t row_bytes = (size_t)(cols / 32) * 34, stored_row_bytes = (size_t)(stored_cols / 32) * 34;
        for (size_t r = 0; r < (size_t)total_rows; ++r)
            std::memcpy(staged.data() + r * stored_row_bytes, p + r * row_bytes, row_bytes);
        p = staged.data();
    }
    FH_HIP(hipSetDevice(device->ordinal));
    void* dptr = nullptr;
    // 16 spare bytes keep vector loads of the last block inside the allocation
    hipError_t e = hipMalloc(&dptr, upload_len + 16);
    if (e != hipSuccess)
        return fail(FH_ERR_ALLOCATION, "hipMalloc(%zu): %s", upload_len, hipGetErrorString(e));
    e = hipMemcpyAsync(dptr, p, upload_len, hipMemcpyHostToDevice, device->stream);
    if (e == hipSuccess) e = hipMemsetAsync(static_cast<uint8_t*>(dptr) + upload_len, 0, 16, device->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(device->stream);
    if (e != hipSuccess) {
        (void)hipFree(dptr);
        return hip_fail(e, "weight upload");
    }
    fh_qmatrix* m = new (std::nothrow) fh_qmatrix();
    if (m == nullptr) {
        (void)hipFree(dptr);
        return fail(FH_ERR_ALLOCATION, "out of host memory");
    }
    m->device = device;
    ++device->handles;
    m->ptr = dptr;
    m->bytes = packed_len;
    m->ggml_type = ggml_type;
    m->rows = rows;
    m->cols = cols;
    m->stored_cols = stored_cols;
    m->experts = experts;
    *out = m;
    return FH_OK;
}

void fh_qmatrix_destroy(fh_qmatrix* matrix) {
    if (matrix == nullptr) return;
    release_memory(matrix->device, matrix->ptr);
    drop_device_handle(matrix->device);
    delete matrix;
}

uint64_t fh_qmatrix_rows(const fh_qmatrix* m) { return m ? m->rows : 0; }
uint64_t fh_qmatrix_columns(const fh_qmatrix* m) { return m ? m->cols : 0; }
uint64_t fh_qmatrix_experts(const fh_qmatrix* m) { return m ? m->experts : 0; }
uint32_t fh_qmatrix_ggml_type(const fh_qmatrix* m) { return m ? m->ggml_type : 0; }
size_t fh_qmatrix_byte_size(const fh_qmatrix* m) { return m ? m->bytes : 0; }
void* fh_qmatrix_device_ptr(fh_qmatrix* m) { return m ? m->ptr : nullptr; }

fh_status fh_dequantize(fh_device* device, const fh_qmatrix* weight, const fh_view* out) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device) return fail(FH_ERR_DEVICE_MISMATCH, "weight belongs to another device");
    const uint64_t rows = weight->rows * weight->experts;
    Range o;
    fh_status st = resolve(device, out, rows * weight->cols, "dequantize output", &o);
    if (st != FH_OK) return st;
    device->last_operation = launch_dequantize(device->stream, weight->ggml_type, weight->ptr, rows, weight->stored_cols,
                                               weight->cols, const_cast<uint8_t*>(o.begin), out->dtype);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_embedding_gather_quantized(fh_device* device, const fh_qmatrix* weight,
                                        const uint32_t* tokens, size_t count, const fh_view* out) {
    if (device && device->capturing) return fail(FH_ERR_SYNCHRONIZATION, "not available while an execution is being recorded");
    if (device == nullptr || weight == nullptr || (tokens == nullptr && count))
        return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device) return fail(FH_ERR_DEVICE_MISMATCH, "weight belongs to another device");
    const uint64_t rows = weight->rows * weight->experts;
    for (size_t i = 0; i < count; ++i)
        if (tokens[i] >= rows)
            return fail(FH_ERR_TOKEN, "token id %u is outside vocabulary of %llu", tokens[i],
                        (unsigned long long)rows);
    if (count == 0) return FH_OK;
    if (!fits_u32((uint64_t)count * weight->cols)) return fail(FH_ERR_SHAPE, "gather size overflow");
    Range o;
    fh_status st = resolve(device, out, (uint64_t)count * weight->cols, "gather output", &o);
    if (st != FH_OK) return st;
    // ids travel through the device scratch (the reference carries them in a tensor)
    size_t need = count * sizeof(uint32_t);
    fh_status sst = ensure_scratch(device, need);
    if (sst != FH_OK) return sst;
    FH_HIP(hipMemcpyAsync(scratch_data(device), tokens, need, hipMemcpyHostToDevice, device->stream));
    FH_HIP(hipStreamSynchronize(device->stream));
    device->last_operation =
        launch_embedding_gather(device->stream, weight->ggml_type, weight->ptr, weight->stored_cols, weight->cols,
                                reinterpret_cast<const uint32_t*>(scratch_data(device)), count,
                                const_cast<uint8_t*>(o.begin), out->dtype);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ---- dense projection --------------------------------------------------------------

namespace {

// `f32_tile_from`: row count from which f32 activations take the f16 tiles; negative = the
// device's gemm_f32_min_rows setting
fh_status project(fh_device* device, const fh_qmatrix* weight, const fh_view* x, uint32_t m,
                  const fh_view* y, bool silu_mul, int64_t f32_tile_from = -1) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device) {
        g_last_error = "weight belongs to another device";
        return FH_ERR_DEVICE_MISMATCH;
    }
    const uint64_t n = weight->rows * weight->experts, k = weight->cols;
    if (m == 0 || k > 0xffffffffull - 32)
        return fail(FH_ERR_SHAPE, "quantized projection requires [M,K] matching [N,K]");
    if (weight->padded()) {
        const fh_qmatrix stored = as_stored(weight);
        PaddedActivations pad(device, weight);
        fh_view px{};
        pad.add(x, (uint64_t)m * (silu_mul ? 2 : 1), "projection input", &px);
        fh_status pst = pad.run();
        if (pst == FH_OK) pst = pad.keep_apart(y, (uint64_t)m * n, "projection output", "projection output aliases its input");
        if (pst != FH_OK) return pst;
        return project(device, &stored, &px, m, y, silu_mul, f32_tile_from);
    }
    const uint64_t x_elements = (uint64_t)m * k * (silu_mul ? 2 : 1);
    if (!fits_u32(x_elements) || !fits_u32((uint64_t)m * n) || !fits_u32(n))
        return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
    Range xr, yr;
    fh_status st = resolve(device, x, x_elements, "projection input", &xr);
    if (st != FH_OK) return st;
    st = resolve(device, y, (uint64_t)m * n, "projection output", &yr);
    if (st != FH_OK) return st;
    if (overlaps(xr, yr)) return fail(FH_ERR_RANGE, "projection output aliases its input");

    // f32 activations stay on exact f32 weights (the GEMV kernel, once per row) unless the
    // caller asks for the tile kernels from some row count on, as the reference's hybrid
    // engine does from 5 rows (HybridModel::project, src/hybrid/engine.rs:3407-3500): the
    // activations are then rounded to f16 into the device scratch first.
    const int64_t f32_tile_rows = f32_tile_from >= 0 ? f32_tile_from : tuning(device, "gemm_f32_min_rows");
    const bool f32_tile = !silu_mul && x->dtype == FH_F32 && f32_tile_rows > 0 && m >= (uint64_t)f32_tile_rows &&
                          ((uintptr_t)xr.begin & 15u) == 0;
    const void* tile_x = xr.begin;
    if (f32_tile) {
        st = ensure_scratch(device, (size_t)m * k * sizeof(uint16_t));
        if (st != FH_OK) return st;
        launch_round_to_f16(device->stream, reinterpret_cast<const float*>(xr.begin),
                            reinterpret_cast<uint16_t*>(scratch_data(device)), (size_t)m * k);
        tile_x = scratch_data(device);
    }
    const bool tile = f32_tile || (!silu_mul && m >= (uint32_t)tuning(device, "gemm_min_rows") && x->dtype != FH_F32);
    if (tile) {
        GemmArgs a{};
        a.ggml_type = weight->ggml_type;
        a.w = weight->ptr;
        a.x = tile_x;
        a.y = const_cast<uint8_t*>(yr.begin);
        a.n = (uint32_t)n;
        a.k = (uint32_t)k;
        a.m = m;
        a.x_dtype = f32_tile ? FH_F16 : x->dtype;
        a.y_dtype = y->dtype;
        a.cu_count = device->props.multiProcessorCount;
        a.wide_min_rows = (int)tuning(device, "gemm_wide_min_rows");
        a.wide_shape = (int)tuning(device, "gemm_wide_shape");
        a.wide32_tile = (int)tuning(device, "gemm_wide32_tile");
        a.skinny_max_rows = (int)tuning(device, "gemm_skinny_max_rows");
        a.rows_resident = tuning(device, "gemm_resident") != 0 && expert_rows_fit_lds((uint32_t)k, 1, 1);
        a.few_tiles_split = tuning(device, "gemm_few_tiles_split") != 0;
        device->last_operation = launch_gemm(device->stream, a);
    } else {
        GemvArgs a{};
        a.ggml_type = weight->ggml_type;
        a.w = weight->ptr;
        a.x = xr.begin;
        a.y = const_cast<uint8_t*>(yr.begin);
        a.n = (uint32_t)n;
        a.k = (uint32_t)k;
        a.m = m;
        a.x_dtype = x->dtype;
        a.y_dtype = y->dtype;
        a.metadata = nullptr;
        a.experts = 1;
        a.ksplit = (int)tuning(device, "k_quant_gemv_ksplit");
        a.stream = (int)tuning(device, "gemv_stream");
        a.stream_own = tuning(device, "gemv_stream_own_loads") != 0;
        a.cu_count = device->props.multiProcessorCount;
        a.x_mode = silu_mul ? kXSiluMul : kXPlain;
        a.x_rows = m;
        const char* name = "";
        st = run_gemv(device, a, &name);
        if (st != FH_OK) return st;
        if (m > 1)
            name = weight->ggml_type == kQ4K   ? "q4_k_gemm"
                   : weight->ggml_type == kQ5K ? "q5_k_gemm"
                   : weight->ggml_type == kQ6K ? "q6_k_gemm"
                   : weight->ggml_type == kQ8_0 ? "q8_0_gemm"
                                                : "iq4_xs_gemm";
        device->last_operation = name;
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_project_quantized(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                               uint32_t m, const fh_view* y) {
    return project(device, weight, x, m, y, false);
}

fh_status fh_project_silu_mul_quantized(fh_device* device, const fh_qmatrix* weight, const fh_view* packed,
                                        uint32_t m, const fh_view* y) {
    return project(device, weight, packed, m, y, true);
}

// fh_project_quantized through the per-row GEMV kernels only, with the kernel's scratch in the
// library's fixed array: no hipMalloc, hipFree or synchronisation on any path.
fh_status fh_project_quantized_no_alloc(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                                        uint32_t m, const fh_view* y) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device) return fail(FH_ERR_DEVICE_MISMATCH, "weight belongs to another device");
    if (device->fixed_scratch == nullptr) return fail(FH_ERR_DISPATCH, "the fixed scratch is not set up");
    if (weight->padded())
        return fail(FH_ERR_SHAPE, "rows of %llu weights are stored padded and need a temporary for the activations: "
                    "fh_project_quantized takes them", (unsigned long long)weight->cols);
    const uint64_t n = weight->rows * weight->experts, k = weight->cols;
    if (m == 0 || k > 0xffffffffull - 32)
        return fail(FH_ERR_SHAPE, "quantized projection requires [M,K] matching [N,K]");
    if (!fits_u32((uint64_t)m * k) || !fits_u32((uint64_t)m * n) || !fits_u32(n) || m > 65535u)
        return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
    Range xr, yr;
    fh_status st = resolve(device, x, (uint64_t)m * k, "projection input", &xr);
    if (st != FH_OK) return st;
    st = resolve(device, y, (uint64_t)m * n, "projection output", &yr);
    if (st != FH_OK) return st;
    if (overlaps(xr, yr)) return fail(FH_ERR_RANGE, "projection output aliases its input");
    GemvArgs a{};
    a.ggml_type = weight->ggml_type;
    a.w = weight->ptr;
    a.x = xr.begin;
    a.y = const_cast<uint8_t*>(yr.begin);
    a.n = (uint32_t)n;
    a.k = (uint32_t)k;
    a.m = m;
    a.x_dtype = x->dtype;
    a.y_dtype = y->dtype;
    a.experts = 1;
    a.ksplit = (int)tuning(device, "k_quant_gemv_ksplit");
    a.stream = (int)tuning(device, "gemv_stream");
    a.stream_own = tuning(device, "gemv_stream_own_loads") != 0;
    a.cu_count = device->props.multiProcessorCount;
    a.x_mode = kXPlain;
    a.x_rows = m;
    const GemvScratch plan = gemv_scratch(a);
    if (plan.segments > 1) {
        const uint64_t counters = (uint64_t)plan.tiles * m;
        const uint64_t partial_bytes = (uint64_t)plan.segments * m * n * sizeof(float);
        if (counters > kFixedCounterWords || partial_bytes > kFixedScratchBytes - kFixedCounterWords * sizeof(uint32_t))
            return fail(FH_ERR_SHAPE,
                        "projection needs %llu counters and %llu bytes of partial sums; the fixed scratch holds %zu and %zu",
                        (unsigned long long)counters, (unsigned long long)partial_bytes, kFixedCounterWords,
                        kFixedScratchBytes - kFixedCounterWords * sizeof(uint32_t));
        uint8_t* const base = static_cast<uint8_t*>(device->fixed_scratch);
        a.counters = reinterpret_cast<uint32_t*>(base);
        a.partials = reinterpret_cast<float*>(base + kFixedCounterWords * sizeof(uint32_t));
    }
    device->last_operation = launch_gemv(device->stream, a);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ---- measurement ----------------------------------------------------------------------

fh_status fh_probe_read(fh_device* device, const fh_qmatrix* weight) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device) return fail(FH_ERR_PARAMETER, "matrix belongs to another device");
    fh_status st = ensure_scratch(device, 0);
    if (st != FH_OK) return st;
    device->last_operation = launch_read_probe(device->stream, weight->ptr, weight->bytes,
                                               reinterpret_cast<uint32_t*>(scratch_data(device)), tuning(device, "probe_read_form"));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_probe_mfma(fh_device* device, uint32_t shape, uint32_t groups, uint32_t iterations, double* flops) {
    if (device == nullptr || flops == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (shape > 2 || groups == 0 || groups > 65535 || iterations == 0)
        return fail(FH_ERR_SHAPE, "mfma probe: shape 0, 1 or 2, 1..65535 workgroups, at least one iteration");
    fh_status st = ensure_scratch(device, (size_t)groups * 256 * sizeof(float));
    if (st != FH_OK) return st;
    device->last_operation = launch_mfma_probe(device->stream, (int)shape, groups, iterations,
                                               reinterpret_cast<float*>(scratch_data(device)), flops);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_probe_coissue(fh_device* device, uint32_t groups, uint32_t iterations, uint32_t mfma,
                           uint32_t valu_rounds) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (groups == 0 || groups > 65535 || iterations == 0 || (mfma == 0 && valu_rounds == 0))
        return fail(FH_ERR_SHAPE, "co-issue probe: 1..65535 workgroups, at least one iteration, something to run");
    fh_status st = ensure_scratch(device, (size_t)groups * 512 * sizeof(float));
    if (st != FH_OK) return st;
    device->last_operation = launch_coissue_probe(device->stream, groups, iterations, mfma, valu_rounds,
                                                  reinterpret_cast<float*>(scratch_data(device)));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ---- mixture of experts -------------------------------------------------------------

fh_status fh_argmax_rows(fh_device* device, const fh_view* logits, uint32_t rows, uint32_t width,
                         const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (rows == 0 || width == 0 || !fits_u32((uint64_t)rows * width))
        return fail(FH_ERR_SHAPE, "argmax requires nonempty [rows,width]");
    if (out == nullptr || out->dtype != FH_F32) return fail(FH_ERR_DTYPE, "argmax output is an f32 carrier of [rows,2]");
    Range lr, orr;
    fh_status st = resolve(device, logits, (uint64_t)rows * width, "argmax input", &lr);
    if (st != FH_OK) return st;
    st = resolve(device, out, (uint64_t)rows * 2, "argmax output", &orr, 4);
    if (st != FH_OK) return st;
    if (overlaps(lr, orr)) return fail(FH_ERR_RANGE, "argmax output aliases its input");
    device->last_operation = launch_argmax_rows(device->stream, lr.begin, logits->dtype, rows, width,
                                                reinterpret_cast<uint32_t*>(const_cast<uint8_t*>(orr.begin)));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_add_rmsnorm(fh_device* device, const fh_view* a, const fh_view* b, const fh_view* weight,
                         uint32_t rows, uint32_t width, float epsilon, const fh_view* residual,
                         const fh_view* normed) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (rows == 0 || width == 0 || width > 0xffffffffu - 256u || !fits_u32((uint64_t)rows * width))
        return fail(FH_ERR_SHAPE, "fused add+RMSNorm requires nonempty [rows,width]");
    if (a == nullptr || b == nullptr || weight == nullptr || residual == nullptr || normed == nullptr)
        return fail(FH_ERR_RANGE, "fused add+RMSNorm: null view");
    if (a->dtype != b->dtype || weight->dtype != a->dtype || residual->dtype != a->dtype || normed->dtype != a->dtype)
        return fail(FH_ERR_SHAPE, "fused add+RMSNorm operands must match");
    if (!std::isfinite(epsilon) || epsilon <= 0.f)
        return fail(FH_ERR_PARAMETER, "epsilon must be finite and positive");
    const uint64_t count = (uint64_t)rows * width;
    Range ar, br, wr, rr, nr;
    fh_status st = resolve(device, a, count, "add+RMSNorm a", &ar);
    if (st != FH_OK) return st;
    if ((st = resolve(device, b, count, "add+RMSNorm b", &br)) != FH_OK) return st;
    if ((st = resolve(device, weight, width, "add+RMSNorm weight", &wr)) != FH_OK) return st;
    if ((st = resolve(device, residual, count, "add+RMSNorm residual", &rr)) != FH_OK) return st;
    if ((st = resolve(device, normed, count, "add+RMSNorm output", &nr)) != FH_OK) return st;
    for (const Range* out : {&rr, &nr}) {
        if (overlaps(*out, ar) || overlaps(*out, br) || overlaps(*out, wr))
            return fail(FH_ERR_RANGE, "add+RMSNorm outputs alias an operand");
    }
    if (overlaps(rr, nr)) return fail(FH_ERR_RANGE, "add+RMSNorm outputs alias each other");
    device->last_operation = launch_add_rmsnorm(device->stream, ar.begin, br.begin, wr.begin,
                                                const_cast<uint8_t*>(rr.begin), const_cast<uint8_t*>(nr.begin), rows,
                                                width, a->dtype, epsilon);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

namespace {

fh_status route(fh_device* device, const fh_view* logits, uint32_t tokens, const fh_view* selection_bias,
                const fh_routing_policy* policy, const fh_view* metadata, bool ranked, const fh_view* gate_x,
                const fh_view* gate_w, uint32_t hidden, const fh_view* shared_gate, const fh_view* ids = nullptr,
                const fh_view* weights = nullptr, RouteTokenArgs* defer = nullptr) {
    if (device == nullptr || policy == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    const fh_routing_policy& p = *policy;
    if (tokens == 0 || p.experts == 0 || p.top_k == 0 || p.top_k > 16 || p.top_k > p.experts ||
        !std::isfinite(p.normalization_epsilon) || p.normalization_epsilon < 0.f ||
        !std::isfinite(p.routed_scaling_factor) || p.routed_scaling_factor <= 0.f)
        return fail(FH_ERR_SHAPE, "invalid sparse routing geometry");
    if (p.experts > 1024) return fail(FH_ERR_SHAPE, "routing supports at most 1024 experts");
    if (!fits_u32((uint64_t)tokens * p.top_k * 3) || !fits_u32((uint64_t)tokens * p.experts))
        return fail(FH_ERR_SHAPE, "expert assignment count overflow");
    Range lr, mr, br{nullptr, 0};
    // the kernel loads logits one element at a time: a chunk of 16-bit logits over an odd number of experts
    // may start at any element
    fh_status st = resolve(device, logits, (uint64_t)tokens * p.experts, "router logits", &lr,
                           logits != nullptr ? dtype_bytes(logits->dtype) : 4);
    if (st != FH_OK) return st == FH_ERR_DEVICE_MISMATCH ? fail(FH_ERR_SHAPE, "invalid sparse routing geometry") : st;
    if (selection_bias != nullptr) {
        if (selection_bias->dtype != FH_F32) return fail(FH_ERR_SHAPE, "invalid sparse routing geometry");
        st = resolve(device, selection_bias, p.experts, "selection bias", &br, 4);
        if (st != FH_OK) return st == FH_ERR_DEVICE_MISMATCH ? fail(FH_ERR_SHAPE, "invalid sparse routing geometry") : st;
    }
    RouteExtras extras;
    extras.rank_order = ranked ? 1u : 0u;
    mr = Range{nullptr, 0};
    if (ids == nullptr) {
        if (metadata == nullptr || metadata->dtype != FH_F32)
            return fail(FH_ERR_DTYPE, "routing metadata must be f32");
        st = resolve(device, metadata, (uint64_t)tokens * p.top_k * 3, "routing metadata", &mr, 4);
        if (st != FH_OK) return st;
        if (overlaps(lr, mr)) return fail(FH_ERR_RANGE, "routing metadata aliases the logits");
    } else {
        // the hybrid engine's layout: ids and weights as two [tokens, top_k] f32 carriers
        if (weights == nullptr || ids->dtype != FH_F32 || weights->dtype != FH_F32)
            return fail(FH_ERR_DTYPE, "route ids and weights are f32 carriers");
        Range ir, wr;
        st = resolve(device, ids, (uint64_t)tokens * p.top_k, "route ids", &ir, 4);
        if (st != FH_OK) return st;
        st = resolve(device, weights, (uint64_t)tokens * p.top_k, "route weights", &wr, 4);
        if (st != FH_OK) return st;
        if (overlaps(lr, ir) || overlaps(lr, wr) || overlaps(ir, wr))
            return fail(FH_ERR_RANGE, "route outputs alias the logits or each other");
        extras.ids_out = reinterpret_cast<float*>(const_cast<uint8_t*>(ir.begin));
        extras.weights_out = reinterpret_cast<float*>(const_cast<uint8_t*>(wr.begin));
    }
    if (shared_gate != nullptr) {
        if (shared_gate->dtype != FH_F32) return fail(FH_ERR_DTYPE, "the shared-expert gate is f32");
        Range gr;
        st = resolve(device, shared_gate, tokens, "shared-expert gate", &gr, 4);
        if (st != FH_OK) return st;
        extras.shared_gate = reinterpret_cast<float*>(const_cast<uint8_t*>(gr.begin));
        if (gate_w != nullptr) {
            if (gate_w->dtype != FH_F32 || gate_x == nullptr || hidden == 0 || !fits_u32((uint64_t)tokens * hidden))
                return fail(FH_ERR_SHAPE, "the shared-expert gate needs x [tokens, hidden] and an f32 vector [hidden]");
            Range xr, wr;
            st = resolve(device, gate_x, (uint64_t)tokens * hidden, "gate activations", &xr);
            if (st != FH_OK) return st;
            st = resolve(device, gate_w, hidden, "gate vector", &wr, 4);
            if (st != FH_OK) return st;
            extras.gate_x = xr.begin;
            extras.gate_x_dtype = gate_x->dtype;
            extras.gate_w = reinterpret_cast<const float*>(wr.begin);
            extras.hidden = hidden;
        }
    }
    if (defer != nullptr) {
        // checked as a launch would be; the projection that follows routes the token itself
        RouteTokenArgs& r = *defer;
        r = RouteTokenArgs{};
        r.logits = lr.begin;
        r.logits_dtype = logits->dtype;
        r.bias = reinterpret_cast<const float*>(br.begin);
        r.metadata = reinterpret_cast<float*>(const_cast<uint8_t*>(mr.begin));
        r.experts = p.experts;
        r.top_k = p.top_k;
        r.sigmoid = p.sigmoid;
        r.normalize = p.normalize_top_k_prob;
        r.eps = p.normalization_epsilon;
        r.scaling = p.routed_scaling_factor;
        r.rank_order = extras.rank_order;
        return FH_OK;
    }
    device->last_operation = launch_moe_route(
        device->stream, lr.begin, logits->dtype, reinterpret_cast<const float*>(br.begin),
        reinterpret_cast<float*>(const_cast<uint8_t*>(mr.begin)), tokens, p, extras);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_moe_route(fh_device* device, const fh_view* logits, uint32_t tokens,
                       const fh_view* selection_bias, const fh_routing_policy* policy,
                       const fh_view* metadata) {
    return route(device, logits, tokens, selection_bias, policy, metadata, false, nullptr, nullptr, 0, nullptr);
}

fh_status fh_moe_route_ranked(fh_device* device, const fh_view* logits, uint32_t tokens,
                              const fh_routing_policy* policy, const fh_view* x, const fh_view* gate_vector,
                              uint32_t hidden, const fh_view* metadata, const fh_view* shared_gate) {
    return route(device, logits, tokens, nullptr, policy, metadata, true, x, gate_vector, hidden, shared_gate);
}

// ---- the hybrid engine's MoE stages over plain id / weight arrays ----------------------

fh_status fh_hybrid_moe_route(fh_device* device, const fh_view* logits, uint32_t tokens,
                              const fh_routing_policy* policy, const fh_view* x, const fh_view* gate_vector,
                              uint32_t hidden, const fh_view* ids, const fh_view* weights,
                              const fh_view* shared_gate) {
    if (ids == nullptr) return fail(FH_ERR_RANGE, "route ids: null view");
    return route(device, logits, tokens, nullptr, policy, nullptr, true, x, gate_vector, hidden, shared_gate, ids,
                 weights);
}

fh_status fh_hybrid_project(fh_device* device, const fh_qmatrix* weight, const fh_view* x, uint32_t m,
                            const fh_view* y, uint32_t exact) {
    // HybridModel::project (src/hybrid/engine.rs:3407-3500): one row and `exact` keep f32
    // weights; 2..4 rows are a batched GEMV, also exact; from 5 rows (MVB_MAX_ROWS + 1,
    // :3584) the rows go through f16 tiles
    const fh_status st = project(device, weight, x, m, y, false, exact ? 0 : 5);
    if (st != FH_OK) return st;
    static const char* const names[4][5] = {
        {"h_mv_q4_k", "h_mv_q5_k", "h_mv_q6_k", "h_mv_q8_0", "h_mv_iq4_xs"},
        {"h_mvb_q4_k", "h_mvb_q5_k", "h_mvb_q6_k", "h_mvb_q8_0", "h_mvb_iq4_xs"},
        {"h_mms_q4_k", "h_mms_q5_k", "h_mms_q6_k", "h_mms_q8_0", "h_mms_iq4_xs"},
        {"h_mm_q4_k", "h_mm_q5_k", "h_mm_q6_k", "h_mm_q8_0", "h_mm_iq4_xs"}};
    const int tier = m == 1 || exact ? 0 : m <= 4 ? 1 : m <= 32 ? 2 : 3;
    const int f = weight->ggml_type == kQ4K ? 0 : weight->ggml_type == kQ5K ? 1 : weight->ggml_type == kQ6K ? 2
                  : weight->ggml_type == kQ8_0 ? 3 : 4;
    device->last_operation = names[tier][f];
    return FH_OK;
}

namespace {

// A shared expert (dense [rows, k] matrix every token also runs) can ride in a routed
// launch: tokens entries more, reading the token rows or rows of its own (x), writing y.
struct SharedExpert {
    const fh_qmatrix* weight = nullptr;
    uint32_t tokens = 0;
    const fh_view* x = nullptr;
    const fh_view* y = nullptr;
};

// The shared expert of a launch on a padded matrix: its matrix as stored, its own activations padded too.
// `parts`: runs of `cols` elements per row of the shared expert's input.
struct PaddedRider {
    fh_qmatrix stored{};
    fh_view x{};
    SharedExpert rider;
    const SharedExpert* get(const SharedExpert* shared) const { return shared != nullptr ? &rider : nullptr; }
};

fh_status pad_rider(PaddedActivations& pad, const fh_qmatrix* weight, const SharedExpert* shared, uint32_t parts,
                    PaddedRider* out) {
    if (shared == nullptr) return FH_OK;
    if (shared->weight == nullptr || shared->y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (shared->weight->cols != weight->cols)
        return fail(FH_ERR_SHAPE, "the shared expert's matrix must have one expert's shape and format");
    out->stored = as_stored(shared->weight);
    out->rider = *shared;
    out->rider.weight = &out->stored;
    if (shared->x != nullptr) {
        pad.add(shared->x, (uint64_t)shared->tokens * parts, "shared expert input", &out->x);
        out->rider.x = &out->x;
    }
    return FH_OK;
}

fh_status hybrid_project_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x, const fh_view* ids,
                            uint32_t routes, uint32_t x_div, const fh_view* y, const SharedExpert* shared) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device || routes == 0 || x_div == 0 || routes % x_div != 0 || ids == nullptr ||
        ids->dtype != FH_F32)
        return fail(FH_ERR_SHAPE, "expert projection geometry");
    if (weight->padded()) {
        const fh_qmatrix stored = as_stored(weight);
        PaddedActivations pad(device, weight);
        PaddedRider pr;
        fh_view px{};
        pad.add(x, (uint64_t)routes / x_div, "expert input", &px);
        fh_status pst = pad_rider(pad, weight, shared, 1, &pr);
        if (pst == FH_OK) pst = pad.run();
        if (pst == FH_OK) pst = pad.keep_apart(y, (uint64_t)routes * weight->rows, "expert output", "expert output aliases an input");
        if (pst == FH_OK && shared != nullptr)
            pst = pad.keep_apart(shared->y, (uint64_t)shared->tokens * weight->rows, "shared expert output",
                                 "shared expert output aliases another tensor");
        if (pst != FH_OK) return pst;
        return hybrid_project_id(device, &stored, &px, ids, routes, x_div, y, pr.get(shared));
    }
    const uint64_t rows = weight->rows, k = weight->cols;
    if (!fits_u32((uint64_t)routes * rows) || !fits_u32((uint64_t)routes / x_div * k))
        return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
    Range xr, ir, yr;
    fh_status st = resolve(device, x, (uint64_t)routes / x_div * k, "expert input", &xr);
    if (st != FH_OK) return st;
    st = resolve(device, ids, routes, "route ids", &ir, 4);
    if (st != FH_OK) return st;
    st = resolve(device, y, (uint64_t)routes * rows, "expert output", &yr);
    if (st != FH_OK) return st;
    if (overlaps(xr, yr) || overlaps(ir, yr)) return fail(FH_ERR_RANGE, "expert output aliases an input");
    Range sxr{nullptr, 0}, syr{nullptr, 0};
    if (shared != nullptr) {
        const fh_qmatrix* sw = shared->weight;
        if (sw == nullptr || shared->y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
        if (sw->device != device) {
            g_last_error = "weight belongs to another device";
            return FH_ERR_DEVICE_MISMATCH;
        }
        if (sw->experts != 1 || sw->rows != rows || sw->cols != k || sw->ggml_type != weight->ggml_type)
            return fail(FH_ERR_SHAPE, "the shared expert's matrix must have one expert's shape and format");
        // without rows of its own the shared expert reads the token rows of x, one per x_div routes
        if (shared->tokens == 0 || (shared->x == nullptr && shared->tokens != routes / x_div) ||
            !fits_u32((uint64_t)routes + shared->tokens) || !fits_u32((uint64_t)shared->tokens * rows) ||
            !fits_u32((uint64_t)shared->tokens * k))
            return fail(FH_ERR_SHAPE, "the shared expert runs once per token");
        if (shared->y->dtype != y->dtype || (shared->x != nullptr && shared->x->dtype != x->dtype))
            return fail(FH_ERR_DTYPE, "the shared expert's tensors differ in dtype from the routed ones");
        st = resolve(device, shared->y, (uint64_t)shared->tokens * rows, "shared expert output", &syr);
        if (st != FH_OK) return st;
        if (shared->x != nullptr) {
            st = resolve(device, shared->x, (uint64_t)shared->tokens * k, "shared expert input", &sxr);
            if (st != FH_OK) return st;
            if (overlaps(sxr, syr) || overlaps(sxr, yr)) return fail(FH_ERR_RANGE, "expert output aliases an input");
        }
        if (overlaps(xr, syr) || overlaps(ir, syr) || overlaps(yr, syr))
            return fail(FH_ERR_RANGE, "shared expert output aliases another tensor");
    }
    GemvArgs a{};
    a.ggml_type = weight->ggml_type;
    a.w = weight->ptr;
    a.x = xr.begin;
    a.y = const_cast<uint8_t*>(yr.begin);
    a.n = (uint32_t)rows;
    a.k = (uint32_t)k;
    a.m = routes;
    a.x_dtype = x->dtype;
    a.y_dtype = y->dtype;
    a.metadata = reinterpret_cast<const float*>(ir.begin);
    a.meta_stride = 1;
    a.experts = (uint32_t)weight->experts;
    a.x_mode = kXDivide;
    a.x_div = x_div;
    a.x_rows = routes / x_div;
    if (shared != nullptr) {
        a.m = routes + shared->tokens;
        a.shared_w = shared->weight->ptr;
        a.shared_rows = shared->tokens;
        a.shared_x = sxr.begin;
        a.shared_y = const_cast<uint8_t*>(syr.begin);
    }
    const char* unused = "";
    st = run_gemv(device, a, &unused);
    if (st != FH_OK) return st;
    device->last_operation = weight->ggml_type == kQ4K     ? "h_mv_id_q4_k"
                             : weight->ggml_type == kQ5K   ? "h_mv_id_q5_k"
                             : weight->ggml_type == kQ6K   ? "h_mv_id_q6_k"
                             : weight->ggml_type == kQ8_0  ? "h_mv_id_q8_0"
                                                           : "h_mv_id_iq4_xs";
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_hybrid_project_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x, const fh_view* ids,
                               uint32_t routes, uint32_t x_div, const fh_view* y) {
    return hybrid_project_id(device, weight, x, ids, routes, x_div, y, nullptr);
}

fh_status fh_hybrid_project_id_with_shared(fh_device* device, const fh_qmatrix* weight,
                                           const fh_qmatrix* shared_weight, const fh_view* x, const fh_view* ids,
                                           uint32_t routes, uint32_t x_div, uint32_t tokens, const fh_view* shared_x,
                                           const fh_view* y, const fh_view* shared_y) {
    if (shared_weight == nullptr || shared_y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    SharedExpert shared;
    shared.weight = shared_weight;
    shared.tokens = tokens;
    shared.x = shared_x;
    shared.y = shared_y;
    return hybrid_project_id(device, weight, x, ids, routes, x_div, y, &shared);
}

fh_status fh_hybrid_moe_map(fh_device* device, const fh_view* ids, uint32_t experts, uint32_t routes,
                            const fh_view* offsets, const fh_view* sorted, const fh_view* position) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (experts == 0 || experts > 1024 || routes == 0) return fail(FH_ERR_SHAPE, "route map needs 1..1024 experts and routes");
    for (const fh_view* v : {ids, offsets, sorted, position})
        if (v == nullptr || v->dtype != FH_F32) return fail(FH_ERR_DTYPE, "route map operands are f32 carriers of u32");
    Range ir, fr, sr, pr;
    fh_status st = resolve(device, ids, routes, "route ids", &ir, 4);
    if (st != FH_OK) return st;
    if ((st = resolve(device, offsets, (uint64_t)experts + 1, "expert offsets", &fr, 4)) != FH_OK) return st;
    if ((st = resolve(device, sorted, routes, "sorted routes", &sr, 4)) != FH_OK) return st;
    if ((st = resolve(device, position, routes, "route positions", &pr, 4)) != FH_OK) return st;
    if (overlaps(ir, fr) || overlaps(ir, sr) || overlaps(ir, pr) || overlaps(fr, sr) || overlaps(fr, pr) ||
        overlaps(sr, pr))
        return fail(FH_ERR_RANGE, "route map operands alias");
    auto words = [](const Range& r) { return reinterpret_cast<uint32_t*>(const_cast<uint8_t*>(r.begin)); };
    device->last_operation = launch_moe_map(device->stream, words(ir), experts, routes, words(fr), words(sr), words(pr));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_hybrid_moe_gather(fh_device* device, const fh_view* x, const fh_view* sorted, uint32_t hidden,
                               uint32_t used, uint32_t routes, const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (hidden == 0 || used == 0 || routes == 0 || routes % used != 0 || !fits_u32((uint64_t)routes * hidden))
        return fail(FH_ERR_SHAPE, "route gather needs [tokens, hidden] and tokens * used routes");
    if (sorted == nullptr || sorted->dtype != FH_F32 || x == nullptr || out == nullptr || out->dtype != x->dtype)
        return fail(FH_ERR_DTYPE, "route gather: sorted is an f32 carrier, output dtype is the input's");
    Range xr, sr, orr;
    fh_status st = resolve(device, x, (uint64_t)routes / used * hidden, "gather input", &xr);
    if (st != FH_OK) return st;
    if ((st = resolve(device, sorted, routes, "sorted routes", &sr, 4)) != FH_OK) return st;
    if ((st = resolve(device, out, (uint64_t)routes * hidden, "gather output", &orr)) != FH_OK) return st;
    if (overlaps(xr, orr) || overlaps(sr, orr)) return fail(FH_ERR_RANGE, "gather output aliases an input");
    device->last_operation = launch_moe_gather_sorted(
        device->stream, xr.begin, reinterpret_cast<const uint32_t*>(sr.begin), const_cast<uint8_t*>(orr.begin), routes,
        used, routes / used, hidden * (uint32_t)dtype_bytes(x->dtype));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

namespace {

fh_status hybrid_project_mm_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                               const fh_view* offsets, uint32_t routes, const fh_view* y,
                               const SharedExpert* shared) {
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (weight->device != device || routes == 0 || weight->experts > 1024 || offsets == nullptr ||
        offsets->dtype != FH_F32 || x == nullptr || y == nullptr)
        return fail(FH_ERR_SHAPE, "expert projection geometry");
    if (weight->padded()) {
        const fh_qmatrix stored = as_stored(weight);
        PaddedActivations pad(device, weight);
        PaddedRider pr;
        fh_view px{};
        pad.add(x, routes, "expert input", &px);
        if (shared != nullptr && shared->x == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
        fh_status pst = pad_rider(pad, weight, shared, 1, &pr);
        if (pst == FH_OK) pst = pad.run();
        if (pst == FH_OK) pst = pad.keep_apart(y, (uint64_t)routes * weight->rows, "expert output", "expert output aliases an input");
        if (pst == FH_OK && shared != nullptr)
            pst = pad.keep_apart(shared->y, (uint64_t)shared->tokens * weight->rows, "shared expert output",
                                 "shared expert output aliases another tensor");
        if (pst != FH_OK) return pst;
        return hybrid_project_mm_id(device, &stored, &px, offsets, routes, y, pr.get(shared));
    }
    const uint64_t rows = weight->rows, k = weight->cols;
    if (!fits_u32((uint64_t)routes * rows) || !fits_u32((uint64_t)routes * k))
        return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
    if ((rows * dtype_bytes(y->dtype)) % 4 != 0) return fail(FH_ERR_SHAPE, "expert output rows must be whole words");
    Range xr, fr, yr;
    fh_status st = resolve(device, x, (uint64_t)routes * k, "expert input", &xr);
    if (st != FH_OK) return st;
    if ((st = resolve(device, offsets, weight->experts + 1, "expert offsets", &fr, 4)) != FH_OK) return st;
    if ((st = resolve(device, y, (uint64_t)routes * rows, "expert output", &yr)) != FH_OK) return st;
    if (overlaps(xr, yr) || overlaps(fr, yr)) return fail(FH_ERR_RANGE, "expert output aliases an input");
    Range sxr{nullptr, 0}, syr{nullptr, 0};
    if (shared != nullptr) {
        const fh_qmatrix* sw = shared->weight;
        if (sw == nullptr || shared->x == nullptr || shared->y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
        if (sw->device != device) {
            g_last_error = "weight belongs to another device";
            return FH_ERR_DEVICE_MISMATCH;
        }
        if (sw->experts != 1 || sw->rows != rows || sw->cols != k || sw->ggml_type != weight->ggml_type)
            return fail(FH_ERR_SHAPE, "the shared expert's matrix must have one expert's shape and format");
        if (shared->tokens == 0 || !fits_u32((uint64_t)shared->tokens * rows) || !fits_u32((uint64_t)shared->tokens * k))
            return fail(FH_ERR_SHAPE, "the shared expert runs once per token");
        if (shared->y->dtype != y->dtype || shared->x->dtype != x->dtype)
            return fail(FH_ERR_DTYPE, "the shared expert's tensors differ in dtype from the routed ones");
        if ((st = resolve(device, shared->x, (uint64_t)shared->tokens * k, "shared expert input", &sxr)) != FH_OK) return st;
        if ((st = resolve(device, shared->y, (uint64_t)shared->tokens * rows, "shared expert output", &syr)) != FH_OK)
            return st;
        if (overlaps(sxr, syr) || overlaps(sxr, yr) || overlaps(xr, syr) || overlaps(fr, syr) || overlaps(yr, syr))
            return fail(FH_ERR_RANGE, "shared expert output aliases another tensor");
        if (!expert_rows_fit_lds((uint32_t)k, routes, (uint32_t)weight->experts)) {
            // rows too wide for the kernel that carries the shared expert: the two run apart
            st = hybrid_project_mm_id(device, weight, x, offsets, routes, y, nullptr);
            if (st != FH_OK) return st;
            return project(device, shared->weight, shared->x, shared->tokens, shared->y, false, 5);
        }
    }
    // the tiles are f16 / bf16, as the reference's h_mm_id kernels make theirs; f32 rows are rounded to f16 first
    const void* tile_x = xr.begin;
    const void* shared_tile_x = sxr.begin;
    if (x->dtype == FH_F32) {
        const size_t shared_elements = shared != nullptr ? (size_t)shared->tokens * k : 0;
        st = ensure_scratch(device, ((size_t)routes * k + shared_elements) * sizeof(uint16_t));
        if (st != FH_OK) return st;
        uint16_t* x16 = reinterpret_cast<uint16_t*>(scratch_data(device));
        launch_round_to_f16(device->stream, reinterpret_cast<const float*>(xr.begin), x16, (size_t)routes * k);
        tile_x = x16;
        if (shared != nullptr) {
            launch_round_to_f16(device->stream, reinterpret_cast<const float*>(sxr.begin), x16 + (size_t)routes * k,
                                shared_elements);
            shared_tile_x = x16 + (size_t)routes * k;
        }
    }
    GemmArgs g{};
    g.ggml_type = weight->ggml_type;
    g.w = weight->ptr;
    g.x = tile_x;
    g.y = const_cast<uint8_t*>(yr.begin);
    g.n = (uint32_t)rows;
    g.k = (uint32_t)k;
    g.m = routes;
    g.x_dtype = x->dtype == FH_F32 ? FH_F16 : x->dtype;
    g.y_dtype = y->dtype;
    g.cu_count = device->props.multiProcessorCount;
    g.experts = (uint32_t)weight->experts;
    g.expert_offsets = reinterpret_cast<const uint32_t*>(fr.begin);
    g.expert_order = nullptr;   // rows are already expert-sorted
    g.weight_ring = tuning(device, "expert_weight_ring") != 0;
    if (shared != nullptr) {
        g.shared_w = shared->weight->ptr;
        g.shared_rows = shared->tokens;
        g.shared_x = shared_tile_x;
        g.shared_y = const_cast<uint8_t*>(syr.begin);
    }
    launch_gemm_skinny(device->stream, g);
    device->last_operation = weight->ggml_type == kQ4K     ? "h_mm_id_q4_k"
                             : weight->ggml_type == kQ5K   ? "h_mm_id_q5_k"
                             : weight->ggml_type == kQ6K   ? "h_mm_id_q6_k"
                             : weight->ggml_type == kQ8_0  ? "h_mm_id_q8_0"
                                                           : "h_mm_id_iq4_xs";
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_hybrid_project_mm_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                                  const fh_view* offsets, uint32_t routes, const fh_view* y) {
    return hybrid_project_mm_id(device, weight, x, offsets, routes, y, nullptr);
}

fh_status fh_hybrid_project_mm_id_with_shared(fh_device* device, const fh_qmatrix* weight,
                                              const fh_qmatrix* shared_weight, const fh_view* x,
                                              const fh_view* offsets, uint32_t routes, uint32_t tokens,
                                              const fh_view* shared_x, const fh_view* y, const fh_view* shared_y) {
    if (shared_weight == nullptr || shared_x == nullptr || shared_y == nullptr)
        return fail(FH_ERR_PARAMETER, "null argument");
    SharedExpert shared;
    shared.weight = shared_weight;
    shared.tokens = tokens;
    shared.x = shared_x;
    shared.y = shared_y;
    return hybrid_project_mm_id(device, weight, x, offsets, routes, y, &shared);
}

fh_status fh_hybrid_moe_combine(fh_device* device, const fh_view* down, const fh_view* weights,
                                const fh_view* position, const fh_view* shared, const fh_view* shared_gate,
                                uint32_t hidden, uint32_t used, uint32_t tokens, const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (hidden == 0 || used == 0 || tokens == 0 || !fits_u32((uint64_t)tokens * used * hidden))
        return fail(FH_ERR_SHAPE, "route combine needs [tokens * used, hidden]");
    for (const fh_view* v : {down, weights, shared, shared_gate, out})
        if (v == nullptr || v->dtype != FH_F32) return fail(FH_ERR_DTYPE, "the hybrid combine works on f32 rows");
    if (position != nullptr && position->dtype != FH_F32) return fail(FH_ERR_DTYPE, "positions are an f32 carrier of u32");
    const uint64_t routes = (uint64_t)tokens * used;
    Range dr, wr, pr{nullptr, 0}, sr, gr, orr;
    fh_status st = resolve(device, down, routes * hidden, "expert rows", &dr);
    if (st != FH_OK) return st;
    if ((st = resolve(device, weights, routes, "route weights", &wr, 4)) != FH_OK) return st;
    if (position != nullptr && (st = resolve(device, position, routes, "route positions", &pr, 4)) != FH_OK) return st;
    if ((st = resolve(device, shared, (uint64_t)tokens * hidden, "shared rows", &sr)) != FH_OK) return st;
    if ((st = resolve(device, shared_gate, tokens, "shared gate", &gr, 4)) != FH_OK) return st;
    if ((st = resolve(device, out, (uint64_t)tokens * hidden, "combine output", &orr)) != FH_OK) return st;
    if (overlaps(dr, orr) || overlaps(wr, orr) || overlaps(sr, orr) || overlaps(gr, orr) ||
        (position != nullptr && overlaps(pr, orr)))
        return fail(FH_ERR_RANGE, "combine output aliases an input");
    device->last_operation = launch_hybrid_combine(
        device->stream, reinterpret_cast<const float*>(dr.begin), reinterpret_cast<const float*>(wr.begin),
        reinterpret_cast<const uint32_t*>(pr.begin), reinterpret_cast<const float*>(sr.begin),
        reinterpret_cast<const float*>(gr.begin), reinterpret_cast<float*>(const_cast<uint8_t*>(orr.begin)), hidden, used,
        tokens, (uint32_t)routes);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_expert_assign(fh_device* device, const fh_view* hidden, uint32_t tokens,
                           uint32_t width, const fh_view* metadata, uint32_t top_k,
                           const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (tokens == 0 || width == 0 || top_k == 0 || metadata == nullptr || metadata->dtype != FH_F32 ||
        !fits_u32((uint64_t)tokens * top_k) || !fits_u32((uint64_t)tokens * top_k * width))
        return fail(FH_ERR_SHAPE, "expert assignments require [S,H] and [S*top_k,3]");
    const uint32_t assignments = tokens * top_k;
    Range hr, mr, orr;
    fh_status st = resolve(device, hidden, (uint64_t)tokens * width, "assign input", &hr);
    if (st != FH_OK) return st;
    st = resolve(device, metadata, (uint64_t)assignments * 3, "assign metadata", &mr, 4);
    if (st != FH_OK) return st;
    st = resolve(device, out, (uint64_t)assignments * width, "assign output", &orr);
    if (st != FH_OK) return st;
    if (out->dtype != hidden->dtype) return fail(FH_ERR_DTYPE, "assign output dtype differs from input");
    if (overlaps(hr, orr) || overlaps(mr, orr)) return fail(FH_ERR_RANGE, "assign output aliases an input");
    device->last_operation = launch_expert_assign(
        device->stream, hr.begin, reinterpret_cast<const float*>(mr.begin),
        const_cast<uint8_t*>(orr.begin), assignments, width * (uint32_t)dtype_bytes(hidden->dtype), tokens);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

namespace {

fh_status expert_project(fh_device* device, const fh_qmatrix* weight, const fh_view* x, uint32_t x_rows,
                         uint32_t form, uint32_t assignments, const fh_view* metadata, const fh_view* y,
                         const SharedExpert* shared = nullptr, const RouteTokenArgs* route = nullptr,
                         bool grouped_before = false) {
    // grouped_before: the grouped form finds offsets and order of these very records (all ids valid)
    // at the head of the scratch, left there by the call before; the scratch must not grow in between
    if (device == nullptr || weight == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (form > FH_INPUT_SILU_MUL) return fail(FH_ERR_PARAMETER, "unknown input form %u", form);
    if (shared != nullptr && form == FH_INPUT_ROWS)
        return fail(FH_ERR_PARAMETER, "a shared expert needs the gathered or the SiLU input form");
    if (form == FH_INPUT_GATHER && x_rows == 0) return fail(FH_ERR_SHAPE, "gathered expert projection needs tokens");
    if (weight->device != device || assignments == 0 || metadata == nullptr ||
        metadata->dtype != FH_F32 || metadata->buffer == nullptr ||
        metadata->buffer->device != device || x == nullptr || x->buffer == nullptr ||
        x->buffer->device != device)
        return fail(FH_ERR_SHAPE, "quantized expert projection geometry mismatch");
    if (weight->padded()) {
        if (route != nullptr || grouped_before)
            return fail(FH_ERR_DISPATCH, "a matrix whose rows are stored padded takes the separate launches");
        if (shared != nullptr && (form == FH_INPUT_SILU_MUL) != (shared->x != nullptr))
            return fail(FH_ERR_PARAMETER, "the shared expert takes its own input in the SiLU form only");
        const fh_qmatrix stored = as_stored(weight);
        PaddedActivations pad(device, weight);
        PaddedRider pr;
        fh_view px{};
        const uint32_t parts = form == FH_INPUT_SILU_MUL ? 2 : 1;
        pad.add(x, form == FH_INPUT_GATHER ? (uint64_t)x_rows : (uint64_t)assignments * parts, "expert input", &px);
        fh_status pst = pad_rider(pad, weight, shared, parts, &pr);
        if (pst == FH_OK) pst = pad.run();
        if (pst == FH_OK)
            pst = pad.keep_apart(y, (uint64_t)assignments * weight->rows, "expert output", "expert output aliases an input");
        if (pst == FH_OK && shared != nullptr)
            pst = pad.keep_apart(shared->y, (uint64_t)shared->tokens * weight->rows, "shared expert output",
                                 "shared expert output aliases another tensor");
        if (pst != FH_OK) return pst;
        return expert_project(device, &stored, &px, x_rows, form, assignments, metadata, y, pr.get(shared));
    }
    const uint64_t rows = weight->rows, k = weight->cols;
    // elements the input view must hold: [A,K], [tokens,K] or [A,2K]
    const uint64_t x_elements = form == FH_INPUT_GATHER ? (uint64_t)x_rows * k
                                : (uint64_t)assignments * k * (form == FH_INPUT_SILU_MUL ? 2 : 1);
    if (!fits_u32((uint64_t)assignments * rows) || !fits_u32(x_elements))
        return fail(FH_ERR_SHAPE, "index does not fit in 32 bits");
    Range xr, mr, yr;
    fh_status st = resolve(device, x, x_elements, "expert input", &xr);
    if (st != FH_OK) return st;
    st = resolve(device, metadata, (uint64_t)assignments * 3, "expert metadata", &mr, 4);
    if (st != FH_OK) return st;
    st = resolve(device, y, (uint64_t)assignments * rows, "expert output", &yr);
    if (st != FH_OK) return st;
    if (overlaps(xr, yr) || overlaps(mr, yr)) return fail(FH_ERR_RANGE, "expert output aliases an input");
    Range sxr{nullptr, 0}, syr{nullptr, 0};
    if (shared != nullptr) {
        const fh_qmatrix* sw = shared->weight;
        if (sw == nullptr || shared->y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
        if (sw->device != device) {
            g_last_error = "weight belongs to another device";
            return FH_ERR_DEVICE_MISMATCH;
        }
        if (sw->experts != 1 || sw->rows != rows || sw->cols != k || sw->ggml_type != weight->ggml_type)
            return fail(FH_ERR_SHAPE, "the shared expert's matrix must have one expert's shape and format");
        if (shared->tokens == 0 || (form == FH_INPUT_GATHER && shared->tokens != x_rows) ||
            !fits_u32((uint64_t)assignments + shared->tokens) || !fits_u32((uint64_t)shared->tokens * rows))
            return fail(FH_ERR_SHAPE, "the shared expert runs once per token");
        if ((form == FH_INPUT_SILU_MUL) != (shared->x != nullptr))
            return fail(FH_ERR_PARAMETER, "the shared expert takes its own input in the SiLU form only");
        if (shared->y->dtype != y->dtype || (shared->x != nullptr && shared->x->dtype != x->dtype))
            return fail(FH_ERR_DTYPE, "the shared expert's tensors differ in dtype from the routed ones");
        st = resolve(device, shared->y, (uint64_t)shared->tokens * rows, "shared expert output", &syr);
        if (st != FH_OK) return st;
        if (shared->x != nullptr) {
            st = resolve(device, shared->x, (uint64_t)shared->tokens * k * 2, "shared expert input", &sxr);
            if (st != FH_OK) return st;
            if (overlaps(sxr, syr) || overlaps(sxr, yr)) return fail(FH_ERR_RANGE, "expert output aliases an input");
        }
        if (overlaps(xr, syr) || overlaps(mr, syr) || overlaps(yr, syr))
            return fail(FH_ERR_RANGE, "shared expert output aliases another tensor");
    }
    const int64_t grouped_min = tuning(device, "expert_grouped_min_assignments");
    // f32 rows join the grouped form when the caller has opted f32 activations into the f16
    // tiles (gemm_f32_min_rows, the hybrid engine's prompt path project_mm_id_in,
    // src/hybrid/engine.rs:3164): they are rounded to f16 into the scratch first
    const int64_t f32_rows = tuning(device, "gemm_f32_min_rows");
    const bool f32_grouped = form == FH_INPUT_ROWS && x->dtype == FH_F32 && f32_rows > 0 &&
                             assignments >= (uint64_t)f32_rows && ((uintptr_t)xr.begin & 15u) == 0;
    const bool grouped = (x->dtype != FH_F32 || f32_grouped) && grouped_min > 0 &&
                         assignments >= (uint64_t)grouped_min && weight->experts <= 1024 &&
                         (rows * dtype_bytes(y->dtype)) % 4 == 0;
    if (grouped && route != nullptr) return fail(FH_ERR_DISPATCH, "only the per-assignment launch routes its token");
    if (grouped && shared != nullptr &&
        !expert_rows_fit_lds((uint32_t)k, assignments, (uint32_t)weight->experts)) {
        // a shared expert rides in the grouped form only in the kernel that keeps rows in LDS;
        // with rows too wide for it the two run apart, as the separate calls would
        st = expert_project(device, weight, x, x_rows, form, assignments, metadata, y, nullptr);
        if (st != FH_OK) return st;
        if (form == FH_INPUT_GATHER) return project(device, shared->weight, x, shared->tokens, shared->y, false);
        if (shared->tokens < (uint64_t)tuning(device, "gemm_min_rows") || ((uintptr_t)sxr.begin & 15u) != 0)
            return project(device, shared->weight, shared->x, shared->tokens, shared->y, true);
        st = ensure_scratch(device, (size_t)shared->tokens * k * sizeof(uint16_t));
        if (st != FH_OK) return st;
        launch_expert_silu_mul(device->stream, sxr.begin, scratch_data(device), shared->tokens, (uint32_t)k, x->dtype,
                               x->dtype);
        GemmArgs g{};
        g.ggml_type = weight->ggml_type;
        g.w = shared->weight->ptr;
        g.x = scratch_data(device);
        g.y = const_cast<uint8_t*>(syr.begin);
        g.n = (uint32_t)rows;
        g.k = (uint32_t)k;
        g.m = shared->tokens;
        g.x_dtype = x->dtype;
        g.y_dtype = y->dtype;
        g.cu_count = device->props.multiProcessorCount;
        g.wide_min_rows = (int)tuning(device, "gemm_wide_min_rows");
        g.wide_shape = (int)tuning(device, "gemm_wide_shape");
        g.wide32_tile = (int)tuning(device, "gemm_wide32_tile");
        g.skinny_max_rows = (int)tuning(device, "gemm_skinny_max_rows");
        g.rows_resident = tuning(device, "gemm_resident") != 0 && expert_rows_fit_lds((uint32_t)k, 1, 1);
        g.few_tiles_split = tuning(device, "gemm_few_tiles_split") != 0;
        device->last_operation = launch_gemm(device->stream, g);
        FH_HIP(hipGetLastError());
        return FH_OK;
    }
    if (grouped) {
        // grouped form: every expert's weights are streamed once for all of its assignments.
        // The kernel that keeps an expert's rows in LDS gathers them from the token rows
        // itself; where they do not fit, and for the SiLU form, the rows are written out
        // first, as the separate expert_assign / expert_silu_mul launches would.
        const bool gathers = form == FH_INPUT_GATHER &&
                             expert_rows_fit_lds((uint32_t)k, assignments, (uint32_t)weight->experts);
        const bool staged = f32_grouped || (form != FH_INPUT_ROWS && !gathers);
        const size_t words = ((size_t)weight->experts + 1 + assignments + 3) & ~(size_t)3;
        // the SiLU form stages the shared expert's rows behind the routed ones
        const size_t staged_rows = (size_t)assignments + (shared != nullptr && form == FH_INPUT_SILU_MUL ? shared->tokens : 0);
        const size_t staged_bytes = staged ? staged_rows * k * sizeof(uint16_t) : 0;
        st = ensure_scratch(device, words * sizeof(uint32_t) + staged_bytes);
        if (st != FH_OK) return st;
        uint32_t* offsets = reinterpret_cast<uint32_t*>(scratch_data(device));
        uint32_t* order = offsets + weight->experts + 1;
        const void* tile_x = xr.begin;
        uint8_t* shared_rows_x = nullptr;  // the shared expert's own rows, when it does not read the token rows
        if (staged) {
            uint8_t* rows_x = scratch_data(device) + words * sizeof(uint32_t);
            if (f32_grouped) {
                launch_round_to_f16(device->stream, reinterpret_cast<const float*>(xr.begin),
                                    reinterpret_cast<uint16_t*>(rows_x), (size_t)assignments * k);
            } else if (form == FH_INPUT_GATHER) {
                launch_expert_assign(device->stream, xr.begin, reinterpret_cast<const float*>(mr.begin), rows_x,
                                     assignments, (uint32_t)(k * sizeof(uint16_t)), x_rows);
            } else if (shared != nullptr) {
                shared_rows_x = rows_x + (size_t)assignments * k * sizeof(uint16_t);
                launch_expert_silu_mul_pair(device->stream, xr.begin, sxr.begin, rows_x, assignments, shared->tokens,
                                            (uint32_t)k, x->dtype);
            } else {
                launch_expert_silu_mul(device->stream, xr.begin, rows_x, assignments, (uint32_t)k, x->dtype,
                                       x->dtype);
            }
            tile_x = rows_x;
        }
        if (!grouped_before)
            launch_expert_group(device->stream, reinterpret_cast<const float*>(mr.begin), assignments,
                                (uint32_t)weight->experts, offsets, order, const_cast<uint8_t*>(yr.begin),
                                (uint32_t)(rows * dtype_bytes(y->dtype)));
        GemmArgs g{};
        g.ggml_type = weight->ggml_type;
        g.w = weight->ptr;
        g.x = tile_x;
        g.y = const_cast<uint8_t*>(yr.begin);
        g.n = (uint32_t)rows;
        g.k = (uint32_t)k;
        g.m = assignments;
        g.x_dtype = f32_grouped ? FH_F16 : x->dtype;
        g.y_dtype = y->dtype;
        g.cu_count = device->props.multiProcessorCount;
        g.experts = (uint32_t)weight->experts;
        g.expert_offsets = offsets;
        g.expert_order = order;
        g.gather_metadata = gathers ? reinterpret_cast<const float*>(mr.begin) : nullptr;
        g.x_rows = x_rows;
        g.weight_ring = tuning(device, "expert_weight_ring") != 0;
        if (shared != nullptr) {
            g.shared_w = shared->weight->ptr;
            g.shared_rows = shared->tokens;
            // gathered form: the token rows themselves, in place or as staged for the routed rows' gather
            g.shared_x = form == FH_INPUT_GATHER ? xr.begin : shared_rows_x;
            g.shared_y = const_cast<uint8_t*>(syr.begin);
        }
        device->last_operation = launch_gemm_skinny(device->stream, g);
        FH_HIP(hipGetLastError());
        return FH_OK;
    }
    GemvArgs a{};
    a.ggml_type = weight->ggml_type;
    a.w = weight->ptr;
    a.x = xr.begin;
    a.y = const_cast<uint8_t*>(yr.begin);
    a.n = (uint32_t)rows;
    a.k = (uint32_t)k;
    a.m = assignments;
    a.x_dtype = x->dtype;
    a.y_dtype = y->dtype;
    a.metadata = reinterpret_cast<const float*>(mr.begin);
    a.experts = (uint32_t)weight->experts;
    a.ksplit = 0;
    a.x_mode = form;
    a.x_rows = form == FH_INPUT_GATHER ? x_rows : assignments;
    a.route = route;
    if (shared != nullptr) {
        a.m = assignments + shared->tokens;
        a.shared_w = shared->weight->ptr;
        a.shared_rows = shared->tokens;
        a.shared_x = sxr.begin;
        a.shared_y = const_cast<uint8_t*>(syr.begin);
    }
    const char* name = "";
    st = run_gemv(device, a, &name);
    if (st != FH_OK) return st;
    device->last_operation = name;
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_expert_project_with_shared(fh_device* device, const fh_qmatrix* weight,
                                        const fh_qmatrix* shared_weight, const fh_view* x, uint32_t tokens,
                                        uint32_t input_form, uint32_t assignments, const fh_view* metadata,
                                        const fh_view* shared_x, const fh_view* y, const fh_view* shared_y) {
    SharedExpert shared;
    shared.weight = shared_weight;
    shared.tokens = tokens;
    shared.x = shared_x;
    shared.y = shared_y;
    if (shared_weight == nullptr || shared_y == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    return expert_project(device, weight, x, tokens, input_form, assignments, metadata, y, &shared);
}

fh_status fh_expert_project_quantized(fh_device* device, const fh_qmatrix* weight,
                                      const fh_view* x, uint32_t assignments,
                                      const fh_view* metadata, const fh_view* y) {
    return expert_project(device, weight, x, assignments, FH_INPUT_ROWS, assignments, metadata, y);
}

fh_status fh_expert_project_fused(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                                  uint32_t x_rows, uint32_t input_form, uint32_t assignments,
                                  const fh_view* metadata, const fh_view* y) {
    return expert_project(device, weight, x, x_rows, input_form, assignments, metadata, y);
}

fh_status fh_expert_silu_mul(fh_device* device, const fh_view* in, uint32_t assignments,
                             uint32_t intermediate, const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (assignments == 0 || intermediate == 0 || !fits_u32((uint64_t)assignments * intermediate * 2))
        return fail(FH_ERR_SHAPE, "packed expert activation geometry mismatch");
    Range ir, orr;
    fh_status st = resolve(device, in, (uint64_t)assignments * intermediate * 2, "silu_mul input", &ir, 4);
    if (st != FH_OK) return st;
    st = resolve(device, out, (uint64_t)assignments * intermediate, "silu_mul output", &orr, 4);
    if (st != FH_OK) return st;
    if (overlaps(ir, orr)) return fail(FH_ERR_RANGE, "silu_mul output aliases its input");
    device->last_operation = launch_expert_silu_mul(device->stream, ir.begin,
                                                    const_cast<uint8_t*>(orr.begin), assignments,
                                                    intermediate, in->dtype, out->dtype);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

namespace {

fh_status combine(fh_device* device, const fh_view* in, const fh_view* metadata, uint32_t tokens, uint32_t hidden,
                  uint32_t top_k, const fh_view* shared, const fh_view* shared_gate, const fh_view* out) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    if (top_k == 0 || hidden == 0 || tokens == 0 || metadata == nullptr || metadata->dtype != FH_F32 ||
        !fits_u32((uint64_t)tokens * top_k * hidden))
        return fail(FH_ERR_SHAPE, "expert combine geometry mismatch");
    Range ir, mr, orr, sr{nullptr, 0}, gr{nullptr, 0};
    fh_status st = resolve(device, in, (uint64_t)tokens * top_k * hidden, "combine input", &ir, 4);
    if (st != FH_OK) return st;
    st = resolve(device, metadata, (uint64_t)tokens * top_k * 3, "combine metadata", &mr, 4);
    if (st != FH_OK) return st;
    st = resolve(device, out, (uint64_t)tokens * hidden, "combine output", &orr, 4);
    if (st != FH_OK) return st;
    if (overlaps(ir, orr) || overlaps(mr, orr)) return fail(FH_ERR_RANGE, "combine output aliases an input");
    if (shared != nullptr) {
        if (shared->dtype != in->dtype) return fail(FH_ERR_DTYPE, "the shared expert's output has the dtype of the routed rows");
        st = resolve(device, shared, (uint64_t)tokens * hidden, "shared expert output", &sr, 4);
        if (st != FH_OK) return st;
        if (overlaps(sr, orr)) return fail(FH_ERR_RANGE, "combine output aliases an input");
        if (shared_gate != nullptr) {
            if (shared_gate->dtype != FH_F32) return fail(FH_ERR_DTYPE, "the shared-expert gate is f32");
            st = resolve(device, shared_gate, tokens, "shared-expert gate", &gr, 4);
            if (st != FH_OK) return st;
        }
    }
    device->last_operation = launch_expert_combine(
        device->stream, ir.begin, reinterpret_cast<const float*>(mr.begin),
        const_cast<uint8_t*>(orr.begin), tokens, hidden, top_k, in->dtype, out->dtype, sr.begin,
        reinterpret_cast<const float*>(gr.begin));
    FH_HIP(hipGetLastError());
    return FH_OK;
}

}  // namespace

fh_status fh_expert_combine(fh_device* device, const fh_view* in, const fh_view* metadata,
                            uint32_t tokens, uint32_t hidden, uint32_t top_k, const fh_view* out) {
    return combine(device, in, metadata, tokens, hidden, top_k, nullptr, nullptr, out);
}

fh_status fh_expert_combine_shared(fh_device* device, const fh_view* in, const fh_view* metadata,
                                   uint32_t tokens, uint32_t hidden, uint32_t top_k, const fh_view* shared,
                                   const fh_view* shared_gate, const fh_view* out) {
    if (shared == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    return combine(device, in, metadata, tokens, hidden, top_k, shared, shared_gate, out);
}

// ---- the routed FFN in one call ------------------------------------------------------------

namespace {

fh_status ensure_workspace(fh_device* d, size_t bytes) {
    return ensure_block(d, d->workspace, bytes, "the routed FFN's workspace");
}

}  // namespace

fh_status fh_moe_ffn(fh_device* device, const fh_view* hidden, const fh_view* router_logits, uint32_t tokens,
                     const fh_view* selection_bias, const fh_routing_policy* policy,
                     const fh_qmatrix* input_experts, const fh_qmatrix* output_experts,
                     const fh_qmatrix* shared_input, const fh_qmatrix* shared_output,
                     const fh_view* shared_gate, const fh_view* out) {
    if (device == nullptr || hidden == nullptr || router_logits == nullptr || policy == nullptr ||
        input_experts == nullptr || output_experts == nullptr || out == nullptr)
        return fail(FH_ERR_PARAMETER, "null argument");
    // SparseMoe::new's geometry checks (src/nn/moe.rs:137-181)
    const uint64_t e = input_experts->experts, two_i = input_experts->rows, h = input_experts->cols;
    if (tokens == 0 || two_i == 0 || two_i % 2 != 0 || output_experts->experts != e || output_experts->rows != h ||
        output_experts->cols * 2 != two_i || policy->experts != e || policy->top_k == 0 || policy->top_k > e ||
        input_experts->device != device || output_experts->device != device)
        return fail(FH_ERR_SHAPE, "invalid sparse expert weight geometry");
    const bool shared = shared_input != nullptr;
    if ((shared_input == nullptr) != (shared_output == nullptr) ||
        (shared && (shared_input->cols != h || shared_output->rows != h || shared_input->rows == 0 ||
                    shared_input->rows != 2 * shared_output->cols || shared_input->experts != 1 ||
                    shared_output->experts != 1 || shared_input->device != device || shared_output->device != device)))
        return fail(FH_ERR_SHAPE, "invalid shared expert weight geometry");
    if (!shared && shared_gate != nullptr) return fail(FH_ERR_PARAMETER, "a shared gate without a shared expert");
    if (out->dtype != hidden->dtype) return fail(FH_ERR_DTYPE, "the routed FFN writes the activation dtype");
    const uint32_t k = policy->top_k, dt = hidden->dtype;
    const size_t es = dtype_bytes(dt), inter = (size_t)two_i / 2, si = shared ? (size_t)shared_output->cols : 0;
    // matrices whose rows are stored padded take the separate launches, each padding its own activations
    const bool stored_padded = input_experts->padded() || output_experts->padded() ||
                               (shared && (shared_input->padded() || shared_output->padded()));
    const bool rides = shared && shared_input->rows == two_i && shared_input->ggml_type == input_experts->ggml_type &&
                       shared_output->ggml_type == output_experts->ggml_type;

    // tokens are taken in chunks whose routing temporaries stay under the limit (src/nn/moe.rs:232-256)
    const size_t per_assignment = (2 * (size_t)h + 3 * inter) * es + 3 * sizeof(float);
    const size_t per_token = per_assignment * k + ((size_t)e + (size_t)h) * es;
    const size_t limit = (size_t)tuning(device, "moe_routing_temporary_limit");
    const uint32_t chunk = (uint32_t)std::min<size_t>(tokens, std::max<size_t>(1, limit / per_token));

    // workspace layout for one chunk
    const size_t a_max = (size_t)chunk * k;
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += align256(bytes);
        return here;
    };
    const size_t meta_at = take(a_max * 3 * sizeof(float));
    const size_t assigned_at = take(a_max * h * es);
    const size_t projected_at = take(a_max * two_i * es);
    const size_t activated_at = take(a_max * inter * es);
    const size_t expert_out_at = take(a_max * h * es);
    const size_t sproj_at = take(shared ? (size_t)chunk * 2 * si * es : 0);
    const size_t sact_at = take(shared ? (size_t)chunk * si * es : 0);
    const size_t sout_at = take(shared ? (size_t)chunk * h * es : 0);
    fh_status st = ensure_workspace(device, at);
    if (st != FH_OK) return st;
    fh_buffer* ws = device->workspace;
    auto view = [&](size_t offset, uint32_t dtype) { return fh_view{ws, offset, dtype}; };

    for (uint32_t start = 0; start < tokens; start += chunk) {
        const uint32_t count = std::min(chunk, tokens - start);
        const uint32_t a = count * k;
        const fh_view x = {hidden->buffer, hidden->offset + (size_t)start * h * es, dt};
        const fh_view logits = {router_logits->buffer,
                                router_logits->offset + (size_t)start * e * dtype_bytes(router_logits->dtype),
                                router_logits->dtype};
        const fh_view y = {out->buffer, out->offset + (size_t)start * h * es, dt};
        fh_view gate{};
        if (shared_gate) gate = {shared_gate->buffer, shared_gate->offset + (size_t)start * sizeof(float), shared_gate->dtype};
        const fh_view meta = view(meta_at, FH_F32), assigned = view(assigned_at, dt), projected = view(projected_at, dt),
                      activated = view(activated_at, dt), expert_out = view(expert_out_at, dt),
                      sproj = view(sproj_at, dt), sact = view(sact_at, dt), sout = view(sout_at, dt);
        // the copy and the activation ride inside the projections: per assignment in decode, in
        // the grouped kernel's gather of an expert's rows beyond it (f32 rows have no grouped form)
        const bool fused = a <= 31 || dt != FH_F32;
        // One token: the down projection of its entries and the weighted sum over them are one
        // launch (the bits of the two; 17.1 against 18.4 us for the 256-expert top-8 FFN with a
        // shared expert).  From two tokens on the two launches are the faster way (22.1 against
        // 23.2 us): the projection's launch stages an entry's activations once for 32 rows, this one
        // once for 8.
        const bool folded = count == 1 && a <= 31 && (!shared || rides) && !stored_padded &&
                            tuning(device, "moe_fold_combine") != 0 &&
                            (!shared_gate || shared_gate->dtype == FH_F32) &&
                            expert_down_combine_fits(output_experts->ggml_type, (uint32_t)h, (uint32_t)inter, k, shared);
        // ... and so does the routing: every workgroup of the gate|up launch routes the token
        // itself before it asks for its expert's rows, which takes a launch and the wait for its
        // records out of the chain
        const int64_t grouped_from = tuning(device, "expert_grouped_min_assignments");
        const bool routes_inside = folded && tuning(device, "moe_fold_route") != 0 &&
                                   (grouped_from <= 0 || a < (uint64_t)grouped_from) &&   // the per-assignment launch
                                   gemv_routes((uint32_t)two_i, (uint32_t)h, (uint32_t)e, k);
        RouteTokenArgs inside{};
        st = route(device, &logits, count, selection_bias, policy, &meta, false, nullptr, nullptr, 0, nullptr, nullptr,
                   nullptr, routes_inside ? &inside : nullptr);
        if (st != FH_OK) return st;
        if (folded) {
            SharedExpert rider;
            rider.weight = shared_input;
            rider.tokens = count;
            rider.x = nullptr;
            rider.y = &sproj;
            st = expert_project(device, input_experts, &x, count, FH_INPUT_GATHER, a, &meta, &projected,
                                shared ? &rider : nullptr, routes_inside ? &inside : nullptr);
            if (st != FH_OK) return st;
            Range yr, gr{nullptr, 0};
            st = resolve(device, &y, (uint64_t)count * h, "routed FFN output", &yr);
            if (st != FH_OK) return st;
            if (shared_gate) {
                st = resolve(device, &gate, count, "shared-expert gate", &gr, 4);
                if (st != FH_OK) return st;
            }
            ExpertDownCombineArgs d{};
            d.ggml_type = output_experts->ggml_type;
            d.w = output_experts->ptr;
            d.w_shared = shared ? shared_output->ptr : nullptr;
            d.x = static_cast<const uint8_t*>(ws->ptr) + projected_at;
            d.x_shared = shared ? static_cast<const uint8_t*>(ws->ptr) + sproj_at : nullptr;
            d.metadata = reinterpret_cast<const float*>(static_cast<const uint8_t*>(ws->ptr) + meta_at);
            d.shared_gate = reinterpret_cast<const float*>(gr.begin);
            d.y = const_cast<uint8_t*>(yr.begin);
            d.n = (uint32_t)h;
            d.k = (uint32_t)inter;
            d.tokens = count;
            d.top_k = k;
            d.experts = (uint32_t)e;
            d.dtype = dt;
            device->last_operation = launch_expert_down_combine(device->stream, d);
            FH_HIP(hipGetLastError());
            continue;
        }
        // Both projections of a chunk group the same records by expert: the second finds the first's
        // offsets and order at the head of the scratch (the router's ids are all valid, and the scratch
        // is brought to the larger call's size before the first, so it does not move in between).
        const int64_t group_from = tuning(device, "expert_grouped_min_assignments");
        // (With a shared expert whose rows do not fit LDS a projection runs the shared matrix as a dense call of its
        // own after the grouping, and that call may put partial sums where the lists lie: both then group for themselves.)
        const bool shared_stays_inside = !shared || (rides && expert_rows_fit_lds((uint32_t)h, a, (uint32_t)e) &&
                                                     expert_rows_fit_lds((uint32_t)inter, a, (uint32_t)e));
        const bool regroup_once = fused && dt != FH_F32 && group_from > 0 && a >= (uint64_t)group_from && e <= 1024 &&
                                  shared_stays_inside && !stored_padded;
        if (regroup_once) {
            const size_t words = ((size_t)e + 1 + a + 3) & ~(size_t)3;
            const size_t widest = std::max<size_t>(h, inter);
            st = ensure_scratch(device, words * sizeof(uint32_t) + ((size_t)a + count) * widest * sizeof(uint16_t));
            if (st != FH_OK) return st;
        }
        if (shared && rides && fused) {
            SharedExpert in_rider, out_rider;
            in_rider.weight = shared_input;
            in_rider.tokens = count;
            in_rider.y = &sproj;
            out_rider.weight = shared_output;
            out_rider.tokens = count;
            out_rider.x = &sproj;
            out_rider.y = &sout;
            st = expert_project(device, input_experts, &x, count, FH_INPUT_GATHER, a, &meta, &projected, &in_rider);
            if (st != FH_OK) return st;
            st = expert_project(device, output_experts, &projected, count, FH_INPUT_SILU_MUL, a, &meta, &expert_out,
                                &out_rider, nullptr, regroup_once);
            if (st != FH_OK) return st;
        } else {
            if (fused) {
                st = expert_project(device, input_experts, &x, count, FH_INPUT_GATHER, a, &meta, &projected);
                if (st != FH_OK) return st;
                st = expert_project(device, output_experts, &projected, a, FH_INPUT_SILU_MUL, a, &meta, &expert_out,
                                    nullptr, nullptr, regroup_once);
                if (st != FH_OK) return st;
            } else {
                st = fh_expert_assign(device, &x, count, (uint32_t)h, &meta, k, &assigned);
                if (st != FH_OK) return st;
                st = fh_expert_project_quantized(device, input_experts, &assigned, a, &meta, &projected);
                if (st != FH_OK) return st;
                st = fh_expert_silu_mul(device, &projected, a, (uint32_t)inter, &activated);
                if (st != FH_OK) return st;
                st = fh_expert_project_quantized(device, output_experts, &activated, a, &meta, &expert_out);
                if (st != FH_OK) return st;
            }
            if (shared) {
                st = fh_project_quantized(device, shared_input, &x, count, &sproj);
                if (st != FH_OK) return st;
                if (count <= 31) {
                    st = fh_project_silu_mul_quantized(device, shared_output, &sproj, count, &sout);
                } else {
                    st = fh_expert_silu_mul(device, &sproj, count, (uint32_t)si, &sact);
                    if (st != FH_OK) return st;
                    st = fh_project_quantized(device, shared_output, &sact, count, &sout);
                }
                if (st != FH_OK) return st;
            }
        }
        st = shared ? fh_expert_combine_shared(device, &expert_out, &meta, count, (uint32_t)h, k, &sout,
                                               shared_gate ? &gate : nullptr, &y)
                    : fh_expert_combine(device, &expert_out, &meta, count, (uint32_t)h, k, &y);
        if (st != FH_OK) return st;
    }
    return FH_OK;
}

// ---- batched execution ---------------------------------------------------------------

fh_status fh_execution_begin(fh_device* device) {
    if (device == nullptr) return fail(FH_ERR_PARAMETER, "null device");
    if (device->capturing) return fail(FH_ERR_DISPATCH, "nested executions are not supported");
    FH_HIP(hipStreamBeginCapture(device->stream, hipStreamCaptureModeThreadLocal));
    device->capturing = true;
    return FH_OK;
}

fh_status fh_execution_end(fh_device* device, fh_graph** out) {
    if (device == nullptr || out == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    *out = nullptr;
    if (!device->capturing) return fail(FH_ERR_DISPATCH, "no execution is being recorded");
    device->capturing = false;
    hipGraph_t graph = nullptr;
    const hipError_t ended = hipStreamEndCapture(device->stream, &graph);
    drain_deferred(device);
    if (ended != hipSuccess) return hip_fail(ended, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return hip_fail(e, "hipGraphInstantiate");
    }
    fh_graph* g = new (std::nothrow) fh_graph();
    if (g == nullptr) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return fail(FH_ERR_ALLOCATION, "out of host memory");
    }
    g->device = device;
    ++device->handles;
    ++device->live_graphs;
    g->graph = graph;
    g->exec = exec;
    *out = g;
    return FH_OK;
}

fh_status fh_graph_launch(fh_graph* graph) {
    if (graph == nullptr) return fail(FH_ERR_PARAMETER, "null graph");
    if (graph->device->closed) return fail(FH_ERR_DEVICE_MISMATCH, "the graph's device has been destroyed");
    if (graph->device->capturing) return fail(FH_ERR_DISPATCH, "cannot replay while recording");
    FH_HIP(hipGraphLaunch(graph->exec, graph->device->stream));
    return FH_OK;
}

void fh_graph_destroy(fh_graph* graph) {
    if (graph == nullptr) return;
    if (!graph->device->closed && graph->device->capturing) {
        graph->device->deferred_graphs.emplace_back(graph->exec, graph->graph);
    } else {
        if (!graph->device->closed) (void)hipStreamSynchronize(graph->device->stream);
        (void)hipGraphExecDestroy(graph->exec);
        (void)hipGraphDestroy(graph->graph);
    }
    if (--graph->device->live_graphs == 0 && !graph->device->capturing) {
        // nothing can replay on the outgrown scratch blocks any more
        for (void* old : graph->device->retired_scratch) release_memory(graph->device, old);
        graph->device->retired_scratch.clear();
    }
    drop_device_handle(graph->device);
    delete graph;
}

// ---- timing ---------------------------------------------------------------------------

fh_status fh_event_create(fh_device* device, fh_event** out) {
    if (device == nullptr || out == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    *out = nullptr;
    fh_event* ev = new (std::nothrow) fh_event();
    if (ev == nullptr) return fail(FH_ERR_ALLOCATION, "out of host memory");
    hipError_t e = hipEventCreate(&ev->event);
    if (e != hipSuccess) {
        delete ev;
        return hip_fail(e, "hipEventCreate");
    }
    ev->device = device;
    ++device->handles;
    *out = ev;
    return FH_OK;
}

void fh_event_destroy(fh_event* event) {
    if (event == nullptr) return;
    (void)hipEventDestroy(event->event);
    drop_device_handle(event->device);
    delete event;
}

fh_status fh_event_record(fh_event* event) {
    if (event == nullptr) return fail(FH_ERR_PARAMETER, "null event");
    if (event->device->closed) return fail(FH_ERR_DEVICE_MISMATCH, "the event's device has been destroyed");
    FH_HIP(hipEventRecord(event->event, event->device->stream));
    return FH_OK;
}

fh_status fh_event_elapsed_ms(fh_event* start, fh_event* stop, float* ms) {
    if (start == nullptr || stop == nullptr || ms == nullptr) return fail(FH_ERR_PARAMETER, "null argument");
    hipError_t e = hipEventSynchronize(stop->event);
    if (e != hipSuccess) return fail(FH_ERR_SYNCHRONIZATION, "event: %s", hipGetErrorString(e));
    FH_HIP(hipEventElapsedTime(ms, start->event, stop->event));
    return FH_OK;
}

}  // extern "C"
