// Queues in HBM and the tt::backend tensor entry points on top of the C ABI (include/ttbfp.h).
#include "backend.hpp"

#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <mutex>
#include <stdexcept>
#include <unordered_map>

#include "../../../include/ttbfp.h"

namespace tt {

namespace {

thread_local std::string g_last_error;

DEVICE_STATUS_CODE fail(const std::string &msg, DEVICE_STATUS_CODE code = DEVICE_STATUS_CODE::RuntimeError)
{
    g_last_error = msg;
    return code;
}

// Status of a C-ABI call -> DEVICE_STATUS_CODE, keeping the library's message.
DEVICE_STATUS_CODE from_abi(std::int32_t st)
{
    if (st == TTBFP_SUCCESS) return DEVICE_STATUS_CODE::Success;
    g_last_error = ttbfp_last_error();
    return st == TTBFP_TIMEOUT_ERROR ? DEVICE_STATUS_CODE::TimeoutError : DEVICE_STATUS_CODE::RuntimeError;
}

#define TT_TRY(expr)                                                  \
    do {                                                              \
        const DEVICE_STATUS_CODE st__ = (expr);                       \
        if (st__ != DEVICE_STATUS_CODE::Success) return st__;         \
    } while (0)

bool plain_float(DataFormat f) { return f == DataFormat::Float32 || f == DataFormat::Float16_b || f == DataFormat::Float16; }
// formats with the 5-bit exponent of IEEE half: they take Float16 sources and read back as Float16
bool a_family(DataFormat f)
{
    return f == DataFormat::Float16 || f == DataFormat::Bfp8 || f == DataFormat::Bfp4 || f == DataFormat::Bfp2;
}
// integer tensors (embedding indices as RawUInt32, int32 / int8 torch tensors as Int32 / Int8: pybuda/pybuda/tensor.py:667-674;
// device_connector.py:204 also names RawUInt8 and RawUInt16 queues): tiled as they are, an integer format pairs with itself only
bool integer_format(DataFormat f)
{
    return f == DataFormat::RawUInt32 || f == DataFormat::RawUInt16 || f == DataFormat::RawUInt8 || f == DataFormat::Int32 ||
           f == DataFormat::UInt16 || f == DataFormat::Int8;
}
bool queue_format_ok(DataFormat f)
{
    return plain_float(f) || a_family(f) || f == DataFormat::Bfp8_b || f == DataFormat::Bfp4_b || f == DataFormat::Bfp2_b || integer_format(f);
}

// One stream per calling thread: the boundary is entered concurrently from pusher, feeder and main
// threads (pybuda/pybuda/device_connector.py:147-175, backend.py:145-189).  `pending` is set when work may be queued on the
// stream and cleared by a wait that succeeded: memory that such work reads or writes must not be recycled before.
struct ThreadStream {
    void *s = nullptr;
    bool pending = false;
    ~ThreadStream()
    {
        if (!s) return;
        ttbfp_stream_synchronize(s, 0);
        ttbfp_stream_destroy(s);
    }
};

ThreadStream &thread_ctx()
{
    thread_local ThreadStream t;
    if (!t.s && ttbfp_stream_create(&t.s) != TTBFP_SUCCESS) t.s = nullptr;
    return t;
}

// the calling thread's stream, for queueing work on it
void *thread_stream()
{
    ThreadStream &t = thread_ctx();
    t.pending = true;
    return t.s;
}

// waits for the thread's stream (timeout_s <= 0: for as long as it takes)
DEVICE_STATUS_CODE sync_thread_stream(int timeout_s)
{
    ThreadStream &t = thread_ctx();
    const DEVICE_STATUS_CODE st = from_abi(ttbfp_stream_synchronize(t.s, timeout_s));
    if (st == DEVICE_STATUS_CODE::Success) t.pending = false;
    return st;
}

// After a failure or a timeout work may still be queued: true once nothing on the thread's stream can touch memory any
// more (the error text of the failure that led here is kept).
bool drain_thread_stream()
{
    ThreadStream &t = thread_ctx();
    if (!t.pending) return true;
    const std::string keep = g_last_error;
    const bool ok = ttbfp_stream_synchronize(t.s, 0) == TTBFP_SUCCESS;
    g_last_error = keep;
    if (ok) t.pending = false;
    return ok;
}

// Reusable blocks of device memory (staging of sources, results and GEMM operands) and of pinned host memory (what
// tilize_tensor / get_output hand out), so that the steady-state push / get path allocates nothing.  Sizes are rounded to
// powers of two up to 64 MiB and to multiples of 16 MiB above, so that a 4 GiB request does not pin 8; blocks that come
// back while the pool already caches `cap` bytes are freed instead of kept.
class BlockPool {
   public:
    using AllocFn = std::int32_t (*)(std::uint64_t, void **);
    using FreeFn = std::int32_t (*)(void *);
    BlockPool(AllocFn a, FreeFn f, std::uint64_t cap) : alloc_(a), free_(f), cap_(cap) {}

    static std::uint64_t rounded(std::uint64_t bytes)
    {
        constexpr std::uint64_t kBig = 64ull << 20, kStep = 16ull << 20;
        if (bytes > kBig) return (bytes + kStep - 1) / kStep * kStep;
        std::uint64_t size = 1 << 16;
        while (size < bytes) size <<= 1;
        return size;
    }
    DEVICE_STATUS_CODE take(std::uint64_t bytes, void **out)
    {
        const std::uint64_t size = rounded(bytes);
        {
            std::lock_guard<std::mutex> l(m_);
            auto &bucket = free_blocks_[size];
            if (!bucket.empty()) {
                *out = bucket.back();
                bucket.pop_back();
                cached_ -= size;
                return DEVICE_STATUS_CODE::Success;
            }
        }
        TT_TRY(from_abi(alloc_(size, out)));
        std::lock_guard<std::mutex> l(m_);
        size_of_[*out] = size;
        allocations_ += 1;
        return DEVICE_STATUS_CODE::Success;
    }
    // true if `p` is one of the pool's blocks (it is then back in the pool, or freed)
    bool give(const void *p)
    {
        if (!p) return false;
        std::uint64_t size;
        {
            std::lock_guard<std::mutex> l(m_);
            auto it = size_of_.find(p);
            if (it == size_of_.end()) return false;
            size = it->second;
            if (cached_ + size <= cap_) {
                free_blocks_[size].push_back(const_cast<void *>(p));
                cached_ += size;
                return true;
            }
            size_of_.erase(it);
        }
        free_(const_cast<void *>(p));
        return true;
    }
    std::uint64_t allocations()
    {
        std::lock_guard<std::mutex> l(m_);
        return allocations_;
    }

   private:
    AllocFn alloc_;
    FreeFn free_;
    std::uint64_t cap_, cached_ = 0, allocations_ = 0;
    std::mutex m_;
    std::map<std::uint64_t, std::vector<void *>> free_blocks_;
    std::unordered_map<const void *, std::uint64_t> size_of_;
};

std::uint64_t pool_cap(const char *env, std::uint64_t fallback)
{
    const char *v = std::getenv(env);
    return v && *v ? std::strtoull(v, nullptr, 10) : fallback;
}

// never destroyed: HIP may be gone when static destructors run
BlockPool &staging()
{
    static BlockPool *pool = new BlockPool(ttbfp_alloc, ttbfp_free, pool_cap("TTBFP_DEVICE_POOL_BYTES", 16ull << 30));
    return *pool;
}
BlockPool &pinned()
{
    static BlockPool *pool = new BlockPool(ttbfp_host_alloc, ttbfp_host_free, pool_cap("TTBFP_HOST_POOL_BYTES", 4ull << 30));
    return *pool;
}

// A staging block for the duration of a call.  It goes back to the pool only once nothing queued on the thread's stream
// can still use it: after an error or a timeout the stream is drained first, and if even that fails the block is leaked
// rather than handed to another thread while the GPU may still write it.
struct Staged {
    void *p = nullptr;
    ~Staged()
    {
        if (p && drain_thread_stream()) staging().give(p);
    }
};

// Host memory handed to the caller by tilize_tensor / get_output / debinarize_tensor / pad_to_buda_shape: pinned blocks
// from the pool, given back by free_tensor.
DEVICE_STATUS_CODE host_block(std::uint64_t bytes, void **out) { return pinned().take(bytes ? bytes : 1, out); }

DEVICE_STATUS_CODE release_host_block(const void *p)
{
    if (!drain_thread_stream()) return DEVICE_STATUS_CODE::RuntimeError;  // a copy into it may be in flight: leak it
    pinned().give(p);  // not one of ours: the caller's tensor, nothing to do
    return DEVICE_STATUS_CODE::Success;
}

// HBM of a queue: buffer b of the grid starts at base + b * pitch and holds the queue's `slots` entries
// one after another, `entry_bytes` each (that buffer's share of an entry).
//
// The mutex guards the ring's bookkeeping only.  A pusher reserves its slots under it, converts into them with the lock
// released, and publishes them under it again, in the order of the reservations (so that entries become visible in the
// order their slots lie in the ring); a reader pins the entries it reads (`readers`) and pop_output waits for that pin,
// so a pusher and a reader of one queue overlap their GPU work, as the reference's callers expect of a boundary they
// enter without the GIL (pybuda/csrc/backend_api/backend_api.cpp:688-701).
struct Queue {
    tt_dram_io_desc desc;
    DataFormat storage = DataFormat::Invalid;  // format of the tiles in HBM: the declared one, or its full-precision stand-in
    ttbfp_queue_layout layout{};
    std::uint8_t *base = nullptr;
    std::uint64_t entry_bytes = 0, pitch = 0;
    std::uint32_t buffers = 1;
    bool row_major = true;  // plain row-major header-less tiles in one buffer
    std::uint32_t slots = 0, wr = 0, rd = 0, count = 0;
    std::uint32_t reserved = 0;                   // entries being written, behind wr + count
    std::uint64_t ticket_next = 0, ticket_done = 0;  // reservations handed out / published
    std::uint32_t readers = 0;                    // get_output calls reading entries right now
    bool consuming = false;                       // a run_matmul owns the oldest entry: it reads it and then pops it
    std::vector<std::uint8_t> poisoned;           // per slot: published without having been written (a push failed)
    std::uint32_t in_flight = 0, max_in_flight = 0;  // conversions running outside the lock, and the most there ever were
    std::uint8_t *slot(std::uint32_t s) const { return base + s * entry_bytes; }  // in buffer 0; the others `pitch` apart
    std::uint64_t span(std::uint32_t entries) const { return (buffers - 1) * pitch + entries * entry_bytes; }
    std::mutex m;
    std::condition_variable cv;
};

std::mutex g_registry_mutex;
std::map<std::string, std::shared_ptr<Queue>> g_registry;

std::string key_of(const tt_dram_io_desc &d) { return d.netlist_path + "/" + d.queue_name; }

std::shared_ptr<Queue> find_queue(const tt_dram_io_desc &d)
{
    std::lock_guard<std::mutex> l(g_registry_mutex);
    auto it = g_registry.find(key_of(d));
    return it == g_registry.end() ? nullptr : it->second;
}

ttbfp_queue_layout layout_of(const tt_dram_io_desc &d)
{
    return {d.bufq_grid_dim_r, d.bufq_grid_dim_c, d.mblock_m, d.mblock_n, d.ublock_rt, d.ublock_ct, d.ublock_order, d.tile_header};
}

// One buffer's share of one entry.
std::uint64_t entry_bytes_of(const tt_dram_io_desc &d, DataFormat storage)
{
    const std::uint32_t shape[4] = {1, d.t, d.rows(), d.cols()};
    const ttbfp_queue_layout l = layout_of(d);
    return ttbfp_queue_buffer_bytes((std::uint8_t)storage, shape, &l);
}

// What a queue holds when the backend ignores the precision of data formats (BackendConfig::ignore_data_format_precision,
// pybuda/csrc/backend_api/backend_api.cpp:261-275: "run backend at full precision"): every format with an 8-bit exponent
// keeps fp32 tiles, the family with the 5-bit exponent of IEEE half keeps the halves it is fed, raw integers stay raw.
DataFormat full_precision_of(DataFormat f)
{
    if (integer_format(f)) return f;
    return a_family(f) ? DataFormat::Float16 : DataFormat::Float32;
}

// Header-less tiles of one buffer in plain row-major order: what the GEMM reads its weight in.
bool row_major_order(const tt_dram_io_desc &d)
{
    if (d.tile_header || d.bufq_grid_dim_r != 1 || d.bufq_grid_dim_c != 1) return false;
    return d.mblock_n == 1 || (d.ublock_rt == 1 && (d.ublock_order == 0 || d.mblock_m == 1));
}

// tilize+pack `wn` entries of a row-major device tensor into slots slot0.. of a queue, and the reverse.
// The memory holds rows x cols per slice (0: as many as the entry has); what lies between that and the entry's
// tile-aligned extent is padding made inside the launch: zeros, or copies of a single row / column (rep_r / rep_c).
DEVICE_STATUS_CODE pack_into(const Queue &q, std::uint32_t slot0, const std::uint8_t *src, DataFormat src_fmt, std::uint32_t wn,
                             const std::uint64_t st[4], void *stream, std::uint32_t rows = 0, std::uint32_t cols = 0, bool rep_r = false,
                             bool rep_c = false)
{
    const std::uint32_t shape[4] = {wn, q.desc.t, rows ? rows : q.desc.rows(), cols ? cols : q.desc.cols()};
    if (shape[2] != q.desc.rows() || shape[3] != q.desc.cols())
        return from_abi(ttbfp_tilize_pack_padded(src, (std::uint8_t)src_fmt, shape, st, rep_r, rep_c, (std::uint8_t)q.storage, conversion_rounding(),
                                                 q.row_major ? nullptr : &q.layout, q.pitch, q.slot(slot0),
                                                 q.row_major ? wn * q.entry_bytes : q.span(wn), stream));
    if (q.row_major)
        return from_abi(ttbfp_tilize_pack(src, (std::uint8_t)src_fmt, shape, st, (std::uint8_t)q.storage,
                                          conversion_rounding(), q.slot(slot0), wn * q.entry_bytes, stream));
    return from_abi(ttbfp_tilize_pack_queue(src, (std::uint8_t)src_fmt, shape, st, (std::uint8_t)q.storage,
                                            conversion_rounding(), &q.layout, q.pitch, q.slot(slot0), q.span(wn), stream));
}

template <typename Pred>
bool wait_until(std::unique_lock<std::mutex> &l, std::condition_variable &cv, int timeout_s, Pred pred)
{
    if (pred()) return true;
    if (timeout_s <= 0) return false;
    return cv.wait_for(l, std::chrono::seconds(timeout_s), pred);
}

// Bytes from the first to one past the last element of a strided tensor.
std::uint64_t span_bytes(const tt_PytorchTensorDesc &t)
{
    std::uint64_t last = 0;
    for (int i = 0; i < 4; ++i) last += (std::uint64_t)(t.shape[i] - 1) * t.strides[i];
    return last + t.itemsize;
}

DEVICE_STATUS_CODE check_source(const tt_PytorchTensorDesc &t, DataFormat dst, const char *fn)
{
    if (!t.ptr) return fail(std::string(fn) + ": tensor descriptor has no data pointer");
    if (integer_format(t.format) || integer_format(dst)) {
        if (t.format != dst)
            return fail(std::string(fn) + ": " + data_format_name(t.format) + " tensor for a " + data_format_name(dst) +
                        " queue: an integer format goes with queues of the same format and nothing else does");
        if (t.itemsize != data_format_byte_size(dst)) return fail(std::string(fn) + ": itemsize does not match the format");
        for (int i = 0; i < 4; ++i)
            if (t.shape[i] == 0) return fail(std::string(fn) + ": empty dimension");
        return DEVICE_STATUS_CODE::Success;
    }
    if (!plain_float(t.format))
        return fail(std::string(fn) + ": source format " + data_format_name(t.format) +
                    " is not supported; a queue with an 8-bit exponent takes Float32 or Float16_b, one with a 5-bit "
                    "exponent Float16 (pybuda/pybuda/device_connector.py:177-201)");
    if (t.itemsize != data_format_byte_size(t.format)) return fail(std::string(fn) + ": itemsize does not match the format");
    if (!queue_format_ok(dst))
        return fail(std::string(fn) + ": queue format " + data_format_name(dst) + " is not supported by this backend");
    if (dst == DataFormat::Float32 && t.format != DataFormat::Float32)
        return fail(std::string(fn) + ": a 16-bit tensor cannot fill a Float32 queue");
    if (a_family(dst) != (t.format == DataFormat::Float16))
        return fail(std::string(fn) + ": " + data_format_name(t.format) + " tensor for a " + data_format_name(dst) +
                    " queue: Float16 tensors go with Float16/Bfp8/Bfp4/Bfp2 queues and nothing else does "
                    "(pybuda/pybuda/device_connector.py:188-192)");
    for (int i = 0; i < 4; ++i)
        if (t.shape[i] == 0) return fail(std::string(fn) + ": empty dimension");
    return DEVICE_STATUS_CODE::Success;
}

// `zn` z slices starting at slice z0 of `wn` entries from slot slot0 on -> row-major memory with byte strides st.
// rows / cols (0: all): only that corner of every slice is written, the narrowing done inside the launch
DEVICE_STATUS_CODE unpack_from(const Queue &q, std::uint32_t slot0, std::uint32_t wn, std::uint32_t z0, std::uint32_t zn, DataFormat dst_fmt,
                               const std::uint64_t st[4], void *dst, void *stream, std::uint32_t rows = 0, std::uint32_t cols = 0)
{
    const std::uint32_t shape[4] = {wn, zn, rows ? rows : q.desc.rows(), cols ? cols : q.desc.cols()};
    const std::uint8_t *src = q.slot(slot0) + z0 * (q.entry_bytes / q.desc.t);  // a buffer holds its z slices one after another
    if (shape[2] != q.desc.rows() || shape[3] != q.desc.cols())
        return from_abi(ttbfp_unpack_untilize_narrow(src, (std::uint8_t)q.storage, shape, q.row_major ? nullptr : &q.layout, q.pitch,
                                                     (std::uint8_t)dst_fmt, st, dst, stream));
    if (q.row_major)
        return from_abi(ttbfp_unpack_untilize(src, (std::uint8_t)q.storage, shape, (std::uint8_t)dst_fmt, st, dst, stream));
    return from_abi(ttbfp_unpack_untilize_queue(src, (std::uint8_t)q.storage, shape, &q.layout, q.pitch,
                                                (std::uint8_t)dst_fmt, st, dst, stream));
}

// ---- the ring's bookkeeping: everything below runs with the queue's mutex held only while it touches these fields ----

struct Reservation {
    std::uint32_t slot0 = 0, n = 0;
    std::uint64_t ticket = 0;
    bool ring = false;
};

// Slots for n entries: the next n free ones of a ring (waits up to timeout_s for space), or slots ram_ptr.. of a RAM.
DEVICE_STATUS_CODE reserve_write(Queue &q, std::uint32_t n, int timeout_s, int ram_ptr, Reservation &r, const char *fn)
{
    std::unique_lock<std::mutex> l(q.m);
    r.n = n;
    r.ring = q.desc.io_type == IO_TYPE::Queue;
    if (r.ring) {
        if (!wait_until(l, q.cv, timeout_s, [&] { return q.slots - q.count - q.reserved >= n; }))
            return fail(std::string(fn) + ": queue '" + q.desc.queue_name + "' is full", DEVICE_STATUS_CODE::TimeoutError);
        r.slot0 = (q.wr + q.reserved) % q.slots;
        r.ticket = q.ticket_next++;
        q.reserved += n;
        for (std::uint32_t i = 0; i < n; ++i) q.poisoned[(r.slot0 + i) % q.slots] = 0;
    } else {
        r.slot0 = ram_ptr < 0 ? 0 : (std::uint32_t)ram_ptr;
        if (r.slot0 + n > q.slots) return fail(std::string(fn) + ": ram pointer past the end of '" + q.desc.queue_name + "'");
    }
    q.in_flight += 1;
    q.max_in_flight = std::max(q.max_in_flight, q.in_flight);
    return DEVICE_STATUS_CODE::Success;
}

// Makes the reserved entries visible, once every earlier reservation has been.  After a failure the slots are given up
// again if nobody reserved behind them; otherwise they have to be published so that the ring stays whole, but they are
// marked as never written: a reader of such an entry gets an error instead of stale bytes, and pop_output releases it
// like any other.
void publish_write(Queue &q, const Reservation &r, bool ok)
{
    std::unique_lock<std::mutex> l(q.m);
    q.in_flight -= 1;
    if (r.ring) {
        q.cv.wait(l, [&] { return q.ticket_done == r.ticket; });
        q.reserved -= r.n;
        const bool last = q.ticket_next == r.ticket + 1;  // nobody has reserved behind these slots
        if (ok || !last) {
            if (!ok)
                for (std::uint32_t i = 0; i < r.n; ++i) q.poisoned[(r.slot0 + i) % q.slots] = 1;
            q.wr = (q.wr + r.n) % q.slots;
            q.count += r.n;
        }
        if (!ok && last) q.ticket_next = r.ticket;  // the rollback hands the ticket back too
        else q.ticket_done += 1;
    } else if (!ok) {
        for (std::uint32_t i = 0; i < r.n; ++i) q.poisoned[r.slot0 + i] = 1;  // a RAM slot that was only partly rewritten
    }
    q.cv.notify_all();
}

// Pins n entries for reading: the oldest n of a ring (waits up to timeout_s for them; rd_ptr >= 0 names the first slot
// instead), or slots rd_ptr.. of a RAM.  consume: the caller will pop the entry it reads (end_consume); only one such
// reader owns the head of a ring at a time, the next one waits for it and then sees the following entry.
DEVICE_STATUS_CODE begin_read(Queue &q, std::uint32_t n, int timeout_s, int rd_ptr, std::uint32_t &slot0, const char *fn, bool consume = false)
{
    std::unique_lock<std::mutex> l(q.m);
    if (q.desc.io_type == IO_TYPE::Queue) {
        if (!wait_until(l, q.cv, timeout_s, [&] { return q.count >= n && !(consume && q.consuming); }))
            return fail(std::string(fn) + ": queue '" + q.desc.queue_name + (q.count >= n ? "' is being consumed" : "' is empty"),
                        DEVICE_STATUS_CODE::TimeoutError);
        slot0 = rd_ptr >= 0 ? (std::uint32_t)rd_ptr % q.slots : q.rd;
    } else {
        slot0 = rd_ptr < 0 ? 0 : (std::uint32_t)rd_ptr;
        if (slot0 + n > q.slots) return fail(std::string(fn) + ": read pointer past the end of '" + q.desc.queue_name + "'");
    }
    for (std::uint32_t i = 0; i < n; ++i)
        if (q.poisoned[(slot0 + i) % q.slots])
            return fail(std::string(fn) + ": entry " + std::to_string((slot0 + i) % q.slots) + " of '" + q.desc.queue_name +
                        "' was never written: the push that reserved it failed (pop_output releases it)");
    if (consume && q.desc.io_type == IO_TYPE::Queue) q.consuming = true;
    q.readers += 1;
    q.in_flight += 1;
    q.max_in_flight = std::max(q.max_in_flight, q.in_flight);
    return DEVICE_STATUS_CODE::Success;
}

void end_read(Queue &q)
{
    std::lock_guard<std::mutex> l(q.m);
    q.readers -= 1;
    q.in_flight -= 1;
    q.cv.notify_all();
}

// End of a consuming read: drops the caller's pin and, with pop, releases the entry it read once no other reader holds
// entries of the ring (as pop_output would).
void end_consume(Queue &q, bool pop)
{
    std::unique_lock<std::mutex> l(q.m);
    q.readers -= 1;
    q.in_flight -= 1;
    if (q.desc.io_type == IO_TYPE::Queue) {
        if (pop) {
            q.cv.wait(l, [&] { return q.readers == 0; });  // readers hold their pin for bounded GPU work only
            q.poisoned[q.rd] = 0;
            q.rd = (q.rd + 1) % q.slots;
            q.count -= 1;
        }
        q.consuming = false;
    }
    q.cv.notify_all();
}

// Releases the oldest n entries of a ring (waits up to timeout_s for them and for readers that still hold them).
DEVICE_STATUS_CODE release_entries(Queue &q, std::uint32_t n, int timeout_s, const char *fn)
{
    std::unique_lock<std::mutex> l(q.m);
    if (!wait_until(l, q.cv, timeout_s, [&] { return q.count >= n && q.readers == 0; }))
        return fail(std::string(fn) + ": queue '" + q.desc.queue_name + (q.count >= n ? "' is being read" : "' is empty"),
                    DEVICE_STATUS_CODE::TimeoutError);
    for (std::uint32_t i = 0; i < n; ++i) q.poisoned[(q.rd + i) % q.slots] = 0;
    q.rd = (q.rd + n) % q.slots;
    q.count -= n;
    q.cv.notify_all();
    return DEVICE_STATUS_CODE::Success;
}

DEVICE_STATUS_CODE stage_source(const tt_PytorchTensorDesc &t, Staged &staged, const std::uint8_t **dev_src, void *stream)
{
    if (ttbfp_pointer_is_device(t.ptr)) {
        // The tensor already lives in HBM.  Which stream produced it is not known here (the descriptor carries a pointer,
        // nothing else) and this thread's stream is not ordered after any other, so wait for all work on the device first:
        // the call then sees the tensor as complete as it would see a host tensor.
        TT_TRY(from_abi(ttbfp_device_synchronize()));
        *dev_src = (const std::uint8_t *)t.ptr;
        return DEVICE_STATUS_CODE::Success;
    }
    const std::uint64_t span = span_bytes(t);
    TT_TRY(staging().take(span, &staged.p));
    TT_TRY(from_abi(ttbfp_memcpy_h2d(staged.p, t.ptr, span, stream)));
    *dev_src = (const std::uint8_t *)staged.p;
    return DEVICE_STATUS_CODE::Success;
}

}  // namespace

int conversion_rounding()
{
    static const int mode = [] {
        const char *v = std::getenv("TTBFP_ROUNDING");
        return (v && (std::strcmp(v, "nearest") == 0 || std::strcmp(v, "1") == 0)) ? TTBFP_ROUND_NEAREST : TTBFP_ROUND_TRUNCATE;
    }();
    return mode;
}

// ---- tt_backend ------------------------------------------------------------------------------

tt_backend::tt_backend(int device, const tt_backend_config &config) : device_(device), config_(config)
{
    static std::mutex m;
    static int counter = 0;
    std::lock_guard<std::mutex> l(m);
    id_ = "hip_backend_" + std::to_string(counter++);
}

std::shared_ptr<tt_backend> tt_backend::create(int device, const tt_backend_config &config)
{
    return std::shared_ptr<tt_backend>(new tt_backend(device, config));
}

tt_backend::~tt_backend() { finish(); }

DEVICE_STATUS_CODE tt_backend::initialize() { return from_abi(ttbfp_init(device_)); }

DEVICE_STATUS_CODE tt_backend::wait_for_idle()
{
    thread_stream();
    return sync_thread_stream(0);
}

DEVICE_STATUS_CODE tt_backend::finish()
{
    DEVICE_STATUS_CODE result = DEVICE_STATUS_CODE::Success;
    for (const std::string &name : queues_) {
        std::shared_ptr<Queue> q;
        {
            std::lock_guard<std::mutex> l(g_registry_mutex);
            auto it = g_registry.find(id_ + "/" + name);
            if (it == g_registry.end()) continue;
            q = it->second;
            g_registry.erase(it);
        }
        if (from_abi(ttbfp_free(q->base)) != DEVICE_STATUS_CODE::Success) result = DEVICE_STATUS_CODE::RuntimeError;
    }
    queues_.clear();
    return result;
}

tt_dram_io_desc tt_backend::create_queue(const std::string &name, DataFormat format, std::uint32_t t, std::uint32_t mblock_m,
                                         std::uint32_t mblock_n, std::uint32_t ublock_rt, std::uint32_t ublock_ct,
                                         std::uint32_t num_slots, IO_TYPE io_type, std::uint32_t input_count, std::uint32_t grid_r,
                                         std::uint32_t grid_c, std::uint32_t ublock_order, bool tile_header)
{
    if (!queue_format_ok(format))
        throw std::runtime_error(std::string("create_queue: format ") + data_format_name(format) + " is not supported");
    if (!t || !mblock_m || !mblock_n || !ublock_rt || !ublock_ct || !num_slots || !input_count || !grid_r || !grid_c)
        throw std::runtime_error("create_queue: zero-sized geometry");
    if (ublock_order > 1) throw std::runtime_error("create_queue: ublock_order is 0 (r) or 1 (c)");
    auto q = std::make_shared<Queue>();
    tt_dram_io_desc &d = q->desc;
    d.netlist_path = id_;
    d.queue_name = name;
    d.bufq_num_slots = num_slots;
    d.bufq_grid_dim_r = grid_r;
    d.bufq_grid_dim_c = grid_c;
    d.ublock_order = ublock_order;
    d.tile_header = tile_header ? 1 : 0;
    d.ublock_rt = ublock_rt;
    d.ublock_ct = ublock_ct;
    d.mblock_m = mblock_m;
    d.mblock_n = mblock_n;
    d.t = t;
    d.input_count = input_count;
    d.bufq_target_format = format;
    d.io_type = io_type;
    q->storage = config_.ignore_data_format_precision ? full_precision_of(format) : format;
    q->layout = layout_of(d);
    q->row_major = row_major_order(d);
    q->buffers = grid_r * grid_c;
    q->entry_bytes = entry_bytes_of(d, q->storage);
    if (q->entry_bytes > 0xffffffffull) throw std::runtime_error("create_queue: one entry exceeds 4 GiB");
    d.bufq_entry_size = (std::uint32_t)q->entry_bytes;
    q->slots = num_slots;
    q->poisoned.assign(num_slots, 0);
    q->pitch = q->entry_bytes * num_slots;
    void *base = nullptr;
    if (ttbfp_alloc(q->pitch * q->buffers, &base) != TTBFP_SUCCESS)
        throw std::runtime_error(std::string("create_queue: ") + ttbfp_last_error());
    q->base = (std::uint8_t *)base;
    // One (address, channel) pair per buffer of the grid.  The reference's pair is 32 + 16 bits wide; an HBM address here
    // has 48 significant bits, so the pair carries all of it: the low 32 bits as the address, the upper 16 as the channel.
    d.bufq_start_addr_channel.clear();
    for (std::uint32_t b = 0; b < q->buffers; ++b) {
        const std::uint64_t addr = (std::uint64_t)(std::uintptr_t)(q->base + b * q->pitch);
        d.bufq_start_addr_channel.push_back({(std::uint32_t)(addr & 0xffffffffu), (std::uint16_t)((addr >> 32) & 0xffffu)});
    }
    {
        std::lock_guard<std::mutex> l(g_registry_mutex);
        if (g_registry.count(key_of(d))) {
            ttbfp_free(base);
            throw std::runtime_error("create_queue: a queue named '" + name + "' already exists");
        }
        g_registry[key_of(d)] = q;
    }
    queues_.push_back(name);
    return d;
}

tt_dram_io_desc tt_backend::get_queue_descriptor(const std::string &name) const
{
    std::lock_guard<std::mutex> l(g_registry_mutex);
    auto it = g_registry.find(id_ + "/" + name);
    if (it == g_registry.end()) throw std::runtime_error("get_queue_descriptor: no queue named '" + name + "'");
    return it->second->desc;
}

DataFormat tt_backend::queue_storage_format(const std::string &name) const
{
    std::lock_guard<std::mutex> l(g_registry_mutex);
    auto it = g_registry.find(id_ + "/" + name);
    if (it == g_registry.end()) throw std::runtime_error("queue_storage_format: no queue named '" + name + "'");
    return it->second->storage;
}

std::uint32_t tt_backend::queue_max_in_flight(const std::string &name) const
{
    std::shared_ptr<Queue> q;
    {
        std::lock_guard<std::mutex> l(g_registry_mutex);
        auto it = g_registry.find(id_ + "/" + name);
        if (it == g_registry.end()) throw std::runtime_error("queue_max_in_flight: no queue named '" + name + "'");
        q = it->second;
    }
    std::lock_guard<std::mutex> l(q->m);
    return q->max_in_flight;
}

std::uint32_t tt_backend::queue_in_flight(const std::string &name) const
{
    std::shared_ptr<Queue> q;
    {
        std::lock_guard<std::mutex> l(g_registry_mutex);
        auto it = g_registry.find(id_ + "/" + name);
        if (it == g_registry.end()) throw std::runtime_error("queue_in_flight: no queue named '" + name + "'");
        q = it->second;
    }
    std::lock_guard<std::mutex> l(q->m);
    return q->in_flight;
}

DEVICE_STATUS_CODE tt_backend::run_matmul(const std::string &in0, const std::string &weight, const std::string &bias,
                                          const std::string &out, bool gelu, int timeout_s, const std::string &approximate)
{
    if (approximate != "none" && approximate != "tanh") return fail("run_matmul: Gelu does not support " + approximate + " approximation mode.");
    const int32_t epilogue = !gelu ? TTBFP_EPILOGUE_NONE : approximate == "tanh" ? TTBFP_EPILOGUE_GELU_TANH : TTBFP_EPILOGUE_GELU;
    auto lookup = [&](const std::string &n) -> std::shared_ptr<Queue> {
        std::lock_guard<std::mutex> l(g_registry_mutex);
        auto it = g_registry.find(id_ + "/" + n);
        return it == g_registry.end() ? nullptr : it->second;
    };
    auto qa = lookup(in0), qw = lookup(weight), qo = lookup(out);
    auto qb = bias.empty() ? nullptr : lookup(bias);
    if (!qa || !qw || !qo || (!bias.empty() && !qb)) return fail("run_matmul: unknown queue name");
    const std::uint32_t M = qa->desc.rows(), K = qa->desc.cols(), N = qw->desc.cols();
    if (qa->desc.t != 1 || qw->desc.t != 1 || qo->desc.t != 1) return fail("run_matmul: t > 1 is not supported");
    if (qw->desc.rows() != K || qo->desc.rows() != M || qo->desc.cols() != N)
        return fail("run_matmul: queue shapes do not form [M,K] x [K,N] -> [M,N]");
    if (qb && (qb->desc.cols() != N || qb->desc.t != 1)) return fail("run_matmul: bias queue must be [32k, N]");
    // Full-precision mode: the queues hold unquantized fp32 tiles and the matmul is evaluated on them as they are.
    const bool full = config_.ignore_data_format_precision;
    if (full) {
        for (const auto &q : {qa, qw, qo, qb})
            if (q && q->storage != DataFormat::Float32) return fail("run_matmul: full-precision mode needs queues with an 8-bit exponent");
    } else {
        if (qw->desc.bufq_target_format != DataFormat::Bfp8_b) return fail("run_matmul: the weight queue must be Bfp8_b");
        if (!qw->row_major)
            return fail("run_matmul: the weight queue must hold header-less tiles in row-major order (grid 1x1 and one-tile-high micro "
                        "blocks in r order, or one micro block per row of the macro block)");
    }
    const std::uint32_t isz = full ? 4 : 2;
    const DataFormat act_fmt = full ? DataFormat::Float32 : DataFormat::Float16_b;

    void *stream = thread_stream();
    Staged x, y, b, w_full, panel;
    TT_TRY(staging().take((std::uint64_t)M * K * isz, &x.p));
    TT_TRY(staging().take((std::uint64_t)M * N * isz, &y.p));

    std::uint32_t in_slot = 0;
    TT_TRY(begin_read(*qa, 1, timeout_s, -1, in_slot, "run_matmul", true));
    struct ReadPin {  // the activation entry is this call's until it ends: popped on success, left in place otherwise
        Queue &q;
        bool pop = false;
        ~ReadPin() { end_consume(q, pop); }
    } pin{*qa};
    {
        const std::uint64_t st[4] = {(std::uint64_t)M * K * isz, (std::uint64_t)M * K * isz, (std::uint64_t)K * isz, isz};
        TT_TRY(unpack_from(*qa, in_slot, 1, 0, 1, act_fmt, st, x.p, stream));
    }
    const void *bias_dev = nullptr;
    if (qb) {
        const std::uint32_t R = qb->desc.rows();
        TT_TRY(staging().take((std::uint64_t)R * N * isz, &b.p));
        const std::uint64_t st[4] = {(std::uint64_t)R * N * isz, (std::uint64_t)R * N * isz, (std::uint64_t)N * isz, isz};
        TT_TRY(unpack_from(*qb, 0, 1, 0, 1, act_fmt, st, b.p, stream));
        bias_dev = b.p;  // row 0 of the tile-padded bias tensor
    }
    if (full) {
        TT_TRY(staging().take((std::uint64_t)K * N * 4, &w_full.p));
        const std::uint64_t st[4] = {(std::uint64_t)K * N * 4, (std::uint64_t)K * N * 4, (std::uint64_t)N * 4, 4};
        TT_TRY(unpack_from(*qw, 0, 1, 0, 1, DataFormat::Float32, st, w_full.p, stream));
        TT_TRY(from_abi(ttbfp_gemm_f32(M, N, K, x.p, w_full.p, bias_dev, epilogue, y.p, stream)));
    } else {
        // scratch for the forms that use it: W converted once into a bf16 panel (many rows), or partial sums of a split over K
        // (shapes with few macro tiles)
        const std::uint64_t panel_bytes = ttbfp_gemm_bfp8b_workspace_bytes(M, N, K);
        if (panel_bytes) TT_TRY(staging().take(panel_bytes, &panel.p));
        TT_TRY(from_abi(ttbfp_gemm_bfp8b_bf16_ws(M, N, K, x.p, qw->base, bias_dev, epilogue, y.p,
                                                 TTBFP_FMT_FLOAT16_B, panel.p, panel_bytes, stream)));
    }
    Reservation r;
    TT_TRY(reserve_write(*qo, 1, timeout_s, 0, r, "run_matmul"));
    const std::uint64_t st[4] = {(std::uint64_t)M * N * isz, (std::uint64_t)M * N * isz, (std::uint64_t)N * isz, isz};
    DEVICE_STATUS_CODE s = pack_into(*qo, r.slot0, (const std::uint8_t *)y.p, act_fmt, 1, st, stream);
    if (s == DEVICE_STATUS_CODE::Success) s = sync_thread_stream(0);
    publish_write(*qo, r, s == DEVICE_STATUS_CODE::Success);
    TT_TRY(s);
    pin.pop = true;
    return DEVICE_STATUS_CODE::Success;
}

// ---- tt::backend free functions ----------------------------------------------------------------

namespace backend {

std::string last_error() { return g_last_error; }

std::uint64_t pool_allocations() { return staging().allocations() + pinned().allocations(); }

DEVICE_STATUS_CODE translate_addresses(tt_dram_io_desc &q)
{
    return find_queue(q) ? DEVICE_STATUS_CODE::Success : fail("translate_addresses: unknown queue '" + q.queue_name + "'");
}

DEVICE_STATUS_CODE push_input(const tt_dram_io_desc &qd, const tt_PytorchTensorDesc &t, const bool push_one,
                              const int timeout_in_seconds, const int ram_ptr, const bool tile_broadcast_r,
                              const bool tile_broadcast_c)
{
    auto q = find_queue(qd);
    if (!q) return fail("push_input: unknown queue '" + qd.queue_name + "'");
    const tt_dram_io_desc &d = q->desc;
    TT_TRY(check_source(t, d.bufq_target_format, "push_input"));
    // A stride in the caller's descriptor asks for the prestriding transform on the way in
    // (pybuda/pybuda/ttdevice.py:1437-1444): the tensor is the [w, C, H, W] activation, the queue entry its
    // rearranged and tile-padded form.
    const int ps = qd.s_descriptor.stride;
    const bool prestride = ps > 0 && !qd.s_descriptor.xy_offsets.empty();
    std::uint32_t ps_rows_cols[2] = {0, 0};
    std::uint64_t ps_bytes = 0;
    // Rows and columns that are not multiples of 32 are padded to the entry's tiles inside the pack launch: zeros, or for a
    // dimension of one that is broadcast to its tile, copies of it (pad_pytorch_tensor_to_buda, pybuda/pybuda/tensor.py:805-877;
    // pad_to_buda_shape, pybuda/csrc/tt_torch_device/tt_device.cpp:153-189).
    std::uint32_t rows = 0, cols = 0;
    if (prestride) {
        if (qd.s_descriptor.xy_offsets.size() != (std::size_t)ps * ps) return fail("push_input: stride descriptor needs stride*stride offsets");
        for (int k = 0; k < ps * ps; ++k)
            if (qd.s_descriptor.xy_offsets[k] != std::make_pair(k % ps, k / ps))
                return fail("push_input: stride descriptor offsets must be [(x, y) for y in range(stride) for x in range(stride)]");
        const std::uint32_t shape[4] = {t.shape[0], t.shape[1], t.shape[2], t.shape[3]};
        ps_bytes = ttbfp_prestride_shape(t.itemsize, shape, (std::uint32_t)ps, ps_rows_cols);
        if (d.t != 1 || ps_rows_cols[0] != d.rows() || ps_rows_cols[1] != d.cols())
            return fail("push_input: prestrided tensor [1," + std::to_string(ps_rows_cols[0]) + "," + std::to_string(ps_rows_cols[1]) +
                        "] does not match queue entry [t=" + std::to_string(d.t) + "," + std::to_string(d.rows()) + "," +
                        std::to_string(d.cols()) + "]");
    } else {
        if (t.shape[1] != d.t || align_up_tile(t.shape[2]) != d.rows() || align_up_tile(t.shape[3]) != d.cols())
            return fail("push_input: tensor [" + std::to_string(t.shape[0]) + "," + std::to_string(t.shape[1]) + "," +
                        std::to_string(t.shape[2]) + "," + std::to_string(t.shape[3]) + "] does not match queue entry [t=" +
                        std::to_string(d.t) + "," + std::to_string(d.rows()) + "," + std::to_string(d.cols()) + "]");
        rows = t.shape[2], cols = t.shape[3];
        if ((tile_broadcast_r && rows != 1) || (tile_broadcast_c && cols != 1))
            return fail("push_input: Trying to broadcast to tile dim a dimension that's not 1");
    }
    const std::uint32_t n = t.shape[0];
    if (push_one && n != 1) return fail("push_input: push_one with " + std::to_string(n) + " entries in the tensor");
    if (n > q->slots) return fail("push_input: tensor holds more entries than the queue has slots");

    Reservation r;
    TT_TRY(reserve_write(*q, n, timeout_in_seconds, ram_ptr, r, "push_input"));
    // from here on the slots are ours: convert into them without the queue's lock, then publish
    auto work = [&]() -> DEVICE_STATUS_CODE {
        void *stream = thread_stream();
        Staged staged, rearranged;
        const std::uint8_t *dev_src = nullptr;
        TT_TRY(stage_source(t, staged, &dev_src, stream));
        const std::uint32_t first = std::min(n, q->slots - r.slot0);  // entries before the ring wraps
        std::uint64_t st[4] = {t.strides[0], t.strides[1], t.strides[2], t.strides[3]};
        if (prestride) {
            const std::uint32_t shape[4] = {t.shape[0], t.shape[1], t.shape[2], t.shape[3]};
            TT_TRY(staging().take(ps_bytes, &rearranged.p));
            TT_TRY(from_abi(ttbfp_prestride(dev_src, t.itemsize, shape, st, (std::uint32_t)ps, rearranged.p, ps_bytes, stream)));
            dev_src = (const std::uint8_t *)rearranged.p;
            st[3] = t.itemsize, st[2] = st[3] * ps_rows_cols[1], st[1] = st[2] * ps_rows_cols[0], st[0] = st[1];
        }
        TT_TRY(pack_into(*q, r.slot0, dev_src, t.format, first, st, stream, rows, cols, tile_broadcast_r, tile_broadcast_c));
        if (first < n)
            TT_TRY(pack_into(*q, 0, dev_src + (std::uint64_t)first * st[0], t.format, n - first, st, stream, rows, cols, tile_broadcast_r,
                             tile_broadcast_c));
        // the time limit of this call is for space in the queue (as in the reference, whose pushes time out on a full
        // queue); the conversion itself is bounded work and is always waited for
        return sync_thread_stream(0);
    };
    const DEVICE_STATUS_CODE s = work();
    publish_write(*q, r, s == DEVICE_STATUS_CODE::Success);
    return s;
}

DEVICE_STATUS_CODE push_input(const tt_dram_io_desc &qd, const tt_TilizedTensorDesc &t, const int timeout_in_seconds,
                              const int ram_ptr)
{
    auto q = find_queue(qd);
    if (!q) return fail("push_input: unknown queue '" + qd.queue_name + "'");
    if (!t.ptr) return fail("push_input: tilized descriptor has no data (load it with debinarize_tensor)");
    if (t.format != q->storage)
        return fail(std::string("push_input: tilized tensor format ") + data_format_name(t.format) + " differs from the format the queue holds, " +
                    data_format_name(q->storage));
    if (t.num_buffers != q->buffers)
        return fail("push_input: tilized tensor has " + std::to_string(t.num_buffers) + " buffers, the queue's grid has " +
                    std::to_string(q->buffers));
    if (t.buf_size_bytes == 0 || t.buf_size_bytes % q->entry_bytes)
        return fail("push_input: tilized tensor is not a whole number of queue entries");
    const std::uint32_t n = (std::uint32_t)(t.buf_size_bytes / q->entry_bytes);
    if (n > q->slots) return fail("push_input: tensor holds more entries than the queue has slots");

    Reservation r;
    TT_TRY(reserve_write(*q, n, timeout_in_seconds, ram_ptr, r, "push_input"));
    auto work = [&]() -> DEVICE_STATUS_CODE {
        void *stream = thread_stream();
        const bool on_device = ttbfp_pointer_is_device(t.ptr);
        if (on_device) TT_TRY(from_abi(ttbfp_device_synchronize()));  // the producer's stream is not known here
        auto copy = on_device ? ttbfp_memcpy_d2d : ttbfp_memcpy_h2d;
        const std::uint32_t first = std::min(n, q->slots - r.slot0);
        for (std::uint32_t b = 0; b < q->buffers; ++b) {  // buffer b of the tensor into buffer b of the queue
            const std::uint8_t *from = (const std::uint8_t *)t.ptr + (std::uint64_t)b * t.buf_size_bytes;
            TT_TRY(from_abi(copy(q->slot(r.slot0) + b * q->pitch, from, first * q->entry_bytes, stream)));
            if (first < n) TT_TRY(from_abi(copy(q->base + b * q->pitch, from + first * q->entry_bytes, (n - first) * q->entry_bytes, stream)));
        }
        return sync_thread_stream(0);
    };
    const DEVICE_STATUS_CODE s = work();
    if (s != DEVICE_STATUS_CODE::Success) drain_thread_stream();  // the caller's memory must not be read after the call returns
    publish_write(*q, r, s == DEVICE_STATUS_CODE::Success);
    return s;
}

DEVICE_STATUS_CODE get_output(const tt_dram_io_desc &qd, tt_PytorchTensorDesc &out, const bool pop_one,
                              const int timeout_in_seconds, const int rd_ptr, const std::uint32_t narrow_r,
                              const std::uint32_t narrow_c)
{
    auto q = find_queue(qd);
    if (!q) return fail("get_output: unknown queue '" + qd.queue_name + "'");
    const tt_dram_io_desc &d = q->desc;
    // Output host transforms travel in the caller's descriptor (pybuda/pybuda/backend.py:294-302):
    // hstack moves groups of `h` consecutive z slices side by side into the columns, vstack stacks
    // groups of `v` below each other into the rows (pybuda/pybuda/op/eval/buda/tm.py:114-137).  With both,
    // stack_row_major says which index runs fastest inside a group of h*v slices (h if set, else v).
    const std::uint32_t hs = std::max<std::uint32_t>(1, qd.hstack_factor), vs = std::max<std::uint32_t>(1, qd.vstack_factor);
    if (d.t % (hs * vs) != 0) return fail("get_output: t is not divisible by hstack_factor * vstack_factor");
    const std::uint32_t n = pop_one ? 1 : d.input_count;
    if (n > q->slots) return fail("get_output: input_count exceeds the queue's slots");
    // narrow_r / narrow_c (0: keep all): only that many rows / columns of every slice are unpacked and copied back, the
    // narrowing of narrow_buda_tensor_to_pytorch (pybuda/pybuda/tensor.py:879-954) done inside the launch
    const std::uint32_t R = narrow_r ? narrow_r : d.rows(), C = narrow_c ? narrow_c : d.cols();
    if (R > d.rows() || C > d.cols() || align_up_tile(R) != d.rows() || align_up_tile(C) != d.cols())
        return fail("get_output: cannot narrow an entry of " + std::to_string(d.rows()) + " x " + std::to_string(d.cols()) + " to " +
                    std::to_string(R) + " x " + std::to_string(C) + " (the tiles must be those of the narrowed shape)");
    const bool narrowed = R != d.rows() || C != d.cols();
    if (narrowed && (hs != 1 || vs != 1)) return fail("get_output: narrowing does not combine with hstack / vstack");

    // Output formats are the ones pybuda turns back into torch tensors (pybuda/pybuda/tensor.py:730-740):
    // Float32 queues read back as Float32, everything with an 8-bit exponent as Float16_b, unless the
    // caller asked for Float32 by presetting the descriptor's format.
    DataFormat of = integer_format(q->storage)          ? q->storage
                    : a_family(q->storage)              ? DataFormat::Float16
                    : out.format == DataFormat::Float32 ? DataFormat::Float32
                    : q->storage == DataFormat::Float32 ? DataFormat::Float32
                                                        : DataFormat::Float16_b;
    const std::uint32_t isz = data_format_byte_size(of);
    const std::uint64_t per_entry = (std::uint64_t)d.t * R * C * isz;
    if (per_entry * n > 0xffffffffull) return fail("get_output: result exceeds the 32-bit strides of the descriptor");

    std::uint32_t slot0 = 0;
    TT_TRY(begin_read(*q, n, timeout_in_seconds, rd_ptr, slot0, "get_output"));
    void *host = nullptr;
    // result [n, t/(h v), R v, C h]: row pitch C h, slice pitch R v rows
    const std::uint64_t row_pitch = (std::uint64_t)C * hs * isz, slice_pitch = (std::uint64_t)R * vs * row_pitch;
    const std::uint64_t st[4] = {per_entry, slice_pitch, row_pitch, isz};
    auto work = [&]() -> DEVICE_STATUS_CODE {
        void *stream = thread_stream();
        Staged dev;
        TT_TRY(staging().take(per_entry * n, &dev.p));
        const std::uint32_t first = std::min(n, q->slots - slot0);
        auto unpack_range = [&](std::uint32_t slot, std::uint32_t entries, std::uint8_t *dst) -> DEVICE_STATUS_CODE {
            if (hs == 1 && vs == 1) return unpack_from(*q, slot, entries, 0, d.t, of, st, dst, stream, R, C);
            // one launch per run of z slices that land at a constant pitch: the fastest index of the group
            const bool h_fast = qd.stack_row_major != 0 || vs == 1;
            const std::uint32_t run = h_fast ? hs : vs, outer = h_fast ? vs : hs;
            const std::uint64_t run_pitch = h_fast ? (std::uint64_t)C * isz : (std::uint64_t)R * row_pitch;
            const std::uint64_t outer_pitch = h_fast ? (std::uint64_t)R * row_pitch : (std::uint64_t)C * isz;
            const std::uint64_t run_st[4] = {0, run_pitch, row_pitch, isz};
            for (std::uint32_t e = 0; e < entries; ++e)
                for (std::uint32_t zo = 0; zo < d.t / (hs * vs); ++zo)
                    for (std::uint32_t o = 0; o < outer; ++o) {
                        const std::uint32_t z0 = (zo * outer + o) * run;
                        DEVICE_STATUS_CODE s = unpack_from(*q, slot + e, 1, z0, run, of, run_st,
                                                           dst + e * per_entry + zo * slice_pitch + o * outer_pitch, stream);
                        if (s != DEVICE_STATUS_CODE::Success) return s;
                    }
            return DEVICE_STATUS_CODE::Success;
        };
        TT_TRY(unpack_range(slot0, first, (std::uint8_t *)dev.p));
        if (first < n) TT_TRY(unpack_range(0, n - first, (std::uint8_t *)dev.p + first * per_entry));
        TT_TRY(host_block(per_entry * n, &host));
        TT_TRY(from_abi(ttbfp_memcpy_d2h(host, dev.p, per_entry * n, stream)));
        return sync_thread_stream(0);  // the time limit is for entries to arrive; reading them is bounded work
    };
    const DEVICE_STATUS_CODE s = work();
    end_read(*q);
    if (s != DEVICE_STATUS_CODE::Success) {
        if (host) release_host_block(host);
        return s;
    }
    out.ptr = host;
    out.itemsize = isz;
    out.format = of;
    out.shape = {n, d.t / (hs * vs), R * vs, C * hs};
    out.strides = {(std::uint32_t)st[0], (std::uint32_t)st[1], (std::uint32_t)st[2], (std::uint32_t)st[3]};
    out.dim = 4;
    out.owner.reset();
    return DEVICE_STATUS_CODE::Success;
}

DEVICE_STATUS_CODE pop_output(const tt_dram_io_desc &qd, const bool pop_one, const int timeout_in_seconds)
{
    auto q = find_queue(qd);
    if (!q) return fail("pop_output: unknown queue '" + qd.queue_name + "'");
    if (q->desc.io_type != IO_TYPE::Queue) return DEVICE_STATUS_CODE::Success;  // nothing to release in a RAM
    return release_entries(*q, pop_one ? 1 : q->desc.input_count, timeout_in_seconds, "pop_output");
}

template <>
DEVICE_STATUS_CODE free_tensor<tt_PytorchTensorDesc>(tt_PytorchTensorDesc &desc)
{
    const DEVICE_STATUS_CODE s = release_host_block(desc.ptr);
    desc.ptr = nullptr;
    desc.owner.reset();
    return s;
}

template <>
DEVICE_STATUS_CODE free_tensor<tt_TilizedTensorDesc>(tt_TilizedTensorDesc &desc)
{
    const DEVICE_STATUS_CODE s = release_host_block(desc.ptr);
    desc.ptr = nullptr;
    return s;
}

tt_TilizedTensorDesc tilize_tensor(const tt_dram_io_desc &qd, const tt_PytorchTensorDesc &t)
{
    auto must = [](DEVICE_STATUS_CODE s) {
        if (s != DEVICE_STATUS_CODE::Success) throw std::runtime_error("tilize_tensor: " + g_last_error);
    };
    // the descriptor of a registered queue tilizes into the format that queue holds (its declared format, or the
    // full-precision stand-in of a backend that ignores data-format precision); any other descriptor into the one it names
    const auto registered = find_queue(qd);
    const DataFormat fmt = registered ? registered->storage : qd.bufq_target_format;
    must(check_source(t, qd.bufq_target_format, "tilize_tensor"));
    const std::uint32_t shape[4] = {t.shape[0], t.shape[1], t.shape[2], t.shape[3]};
    if (ttbfp_packed_size((std::uint8_t)fmt, shape) == 0)
        must(fail("rows and columns must be multiples of 32 (pad with pad_pytorch_tensor_to_buda first)"));
    // A descriptor that says nothing about geometry (one tile, the default) stands for one buffer of
    // header-less tiles in row-major order; any other must describe the tensor it is given.
    ttbfp_queue_layout lay = layout_of(qd);
    const bool no_geometry = qd.rows() == 32 && qd.cols() == 32 && qd.t == 1 && !qd.tile_header;
    if (no_geometry) lay = {1, 1, shape[2] / 32, shape[3] / 32, 1, 1, 0, 0};
    else if (qd.t != shape[1] || qd.rows() != shape[2] || qd.cols() != shape[3])
        must(fail("tensor [t=" + std::to_string(shape[1]) + "," + std::to_string(shape[2]) + "," + std::to_string(shape[3]) +
                  "] does not match the descriptor's entry [t=" + std::to_string(qd.t) + "," + std::to_string(qd.rows()) + "," +
                  std::to_string(qd.cols()) + "]"));
    const std::uint32_t buffers = lay.grid_r * lay.grid_c;
    const std::uint64_t per_buffer = ttbfp_queue_buffer_bytes((std::uint8_t)fmt, shape, &lay), bytes = per_buffer * buffers;
    if (per_buffer == 0 || per_buffer > 0xffffffffull) must(fail("tilized size does not fit the descriptor (one buffer is limited to 4 GiB)"));
    void *stream = thread_stream();
    void *host = nullptr;
    try {
        Staged src, dst;
        const std::uint8_t *dev_src = nullptr;
        must(stage_source(t, src, &dev_src, stream));
        must(staging().take(bytes, &dst.p));
        const std::uint64_t st[4] = {t.strides[0], t.strides[1], t.strides[2], t.strides[3]};
        must(from_abi(ttbfp_tilize_pack_queue(dev_src, (std::uint8_t)t.format, shape, st, (std::uint8_t)fmt, conversion_rounding(), &lay,
                                              per_buffer, dst.p, bytes, stream)));
        must(host_block(bytes, &host));
        must(from_abi(ttbfp_memcpy_d2h(host, dst.p, bytes, stream)));
        must(sync_thread_stream(0));
    } catch (...) {
        if (host) release_host_block(host);  // drains the stream first
        throw;
    }
    return tt_TilizedTensorDesc(host, buffers, (std::uint32_t)per_buffer, fmt);
}

// The C++ caller's padding (pybuda/csrc/tt_torch_device/tt_device.cpp:153-189): a tensor of up to four dimensions becomes
// 4-D (leading ones), its rows and columns are rounded up to whole tiles (align_up_tile, tt_device.hpp:205-210) and filled
// with zeros, and the result is contiguous.  The result lives in backend-owned pinned memory (free_tensor releases it).
// push_input does not need this step - it pads inside its pack launch - so this is for callers that want the padded
// tensor itself.
tt_PytorchTensorDesc pad_to_buda_shape(const tt_PytorchTensorDesc &t)
{
    if (!t.ptr) throw std::runtime_error("pad_to_buda_shape: tensor descriptor has no data pointer");
    if (ttbfp_pointer_is_device(t.ptr)) throw std::runtime_error("pad_to_buda_shape: the tensor must be in host memory");
    if (t.itemsize == 0 || t.itemsize > 8) throw std::runtime_error("pad_to_buda_shape: bad itemsize");
    const std::uint32_t R = align_up_tile(t.shape[2]), C = align_up_tile(t.shape[3]);
    const std::uint64_t row = (std::uint64_t)C * t.itemsize, slice = row * R, bytes = slice * t.shape[0] * t.shape[1];
    if (bytes > 0xffffffffull) throw std::runtime_error("pad_to_buda_shape: result exceeds the 32-bit strides of the descriptor");
    void *host = nullptr;
    if (host_block(bytes, &host) != DEVICE_STATUS_CODE::Success) throw std::runtime_error("pad_to_buda_shape: " + g_last_error);
    std::memset(host, 0, bytes);
    for (std::uint32_t w = 0; w < t.shape[0]; ++w)
        for (std::uint32_t z = 0; z < t.shape[1]; ++z)
            for (std::uint32_t r = 0; r < t.shape[2]; ++r) {
                const std::uint8_t *src = (const std::uint8_t *)t.ptr + (std::uint64_t)w * t.strides[0] + (std::uint64_t)z * t.strides[1] +
                                          (std::uint64_t)r * t.strides[2];
                std::uint8_t *dst = (std::uint8_t *)host + ((std::uint64_t)w * t.shape[1] + z) * slice + r * row;
                if (t.strides[3] == t.itemsize) {
                    std::memcpy(dst, src, (std::size_t)t.shape[3] * t.itemsize);
                } else {
                    for (std::uint32_t c = 0; c < t.shape[3]; ++c)
                        std::memcpy(dst + (std::size_t)c * t.itemsize, src + (std::uint64_t)c * t.strides[3], t.itemsize);
                }
            }
    return tt_PytorchTensorDesc(host, t.itemsize, t.format, {t.shape[0], t.shape[1], R, C},
                                {(std::uint32_t)(slice * t.shape[1]), (std::uint32_t)slice, (std::uint32_t)row, t.itemsize}, 4);
}

namespace {

void write_file(const void *p, std::uint64_t bytes, const std::string &path)
{
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    if (!f) throw std::runtime_error("binarize_tensor: cannot open " + path);
    f.write((const char *)p, (std::streamsize)bytes);
    if (!f) throw std::runtime_error("binarize_tensor: short write to " + path);
}

void *read_file(std::uint64_t bytes, const std::string &path)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw std::runtime_error("debinarize_tensor: cannot open " + path);
    if ((std::uint64_t)f.tellg() != bytes)
        throw std::runtime_error("debinarize_tensor: " + path + " holds " + std::to_string((std::uint64_t)f.tellg()) +
                                 " bytes, the descriptor needs " + std::to_string(bytes));
    f.seekg(0);
    void *host = nullptr;
    if (host_block(bytes, &host) != DEVICE_STATUS_CODE::Success) throw std::runtime_error("debinarize_tensor: " + g_last_error);
    f.read((char *)host, (std::streamsize)bytes);
    return host;
}

}  // namespace

// The payload only; shape/format metadata travels separately (pybuda/pybuda/tti/archive.py:83-147).
template <>
void binarize_tensor<tt_PytorchTensorDesc>(const tt_PytorchTensorDesc &d, std::string path)
{
    if (span_bytes(d) != d.elements() * d.itemsize) throw std::runtime_error("binarize_tensor: tensor must be contiguous");
    write_file(d.ptr, d.elements() * d.itemsize, path);
}

template <>
void binarize_tensor<tt_TilizedTensorDesc>(const tt_TilizedTensorDesc &d, std::string path)
{
    write_file(d.ptr, (std::uint64_t)d.num_buffers * d.buf_size_bytes, path);
}

template <>
void debinarize_tensor<tt_PytorchTensorDesc>(tt_PytorchTensorDesc &d, std::string path)
{
    d.ptr = read_file(d.elements() * d.itemsize, path);
    d.owner.reset();
}

template <>
void debinarize_tensor<tt_TilizedTensorDesc>(tt_TilizedTensorDesc &d, std::string path)
{
    d.ptr = read_file((std::uint64_t)d.num_buffers * d.buf_size_bytes, path);
}

std::uint32_t get_io_size_in_bytes(DataFormat df, bool is_untilized, std::uint32_t ublock_ct, std::uint32_t ublock_rt,
                                   std::uint32_t mblock_m, std::uint32_t mblock_n, std::uint32_t t, std::uint32_t entries,
                                   std::uint32_t tile_height, std::uint32_t tile_width)
{
    constexpr std::uint64_t kQueueHeader = 32;
    const std::uint64_t tiles = (std::uint64_t)ublock_ct * ublock_rt * mblock_m * mblock_n * t;
    std::uint64_t per_entry;
    if (is_untilized)
        per_entry = tiles * data_format_byte_size(df, (int)(tile_height * tile_width));
    else
        per_entry = tiles * (data_format_byte_size(df, (int)(tile_height * tile_width)) + 32);
    const std::uint64_t total = kQueueHeader + per_entry * entries;
    if (total > 0xffffffffull) throw std::runtime_error("get_io_size_in_bytes: size exceeds 32 bits");
    return (std::uint32_t)total;
}

}  // namespace backend
}  // namespace tt
