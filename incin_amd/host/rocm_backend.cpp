// See rocm_backend.hpp.  Everything that touches the device goes through the C ABI.
#include "rocm_backend.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>

#include "../../include/incin_rocm.h"

namespace incin_rocm_host {

namespace {

thread_local int64_t g_launches = 0;

Error ok() { return Error{}; }
Error err(ErrorKind k, std::string m) { return Error{k, std::move(m)}; }

std::string shape_str(const std::vector<int64_t>& s)
{
    std::string r = "[";
    for (size_t i = 0; i < s.size(); ++i) r += (i ? ", " : "") + std::to_string(s[i]);
    return r + "]";
}

// Status code of the C ABI -> the Error variant the Rust backend would return.
Error from_status(int rc, int32_t device)
{
    if (rc == INCIN_ROCM_OK) return ok();
    const std::string msg = incin_rocm_last_error();
    switch (rc) {
        case INCIN_ROCM_ESHAPE: return err(ErrorKind::ShapeMismatch, msg);
        case INCIN_ROCM_EDTYPE: return err(ErrorKind::UnsupportedDType, msg);
        case INCIN_ROCM_EDEVICE: return err(ErrorKind::InvalidDeviceOrdinal, "backend Rocm, ordinal " + std::to_string(device) + ": " + msg);
        case INCIN_ROCM_ENOMEM: return err(ErrorKind::OutOfMemory, msg);
        case INCIN_ROCM_EUNSUPPORTED: return err(ErrorKind::UnsupportedBackendOperation, msg);
        default: return err(ErrorKind::Msg, msg);
    }
}

// ---- the calling thread's stream, its recording, and the buffer pools ---------------------------------------------------
thread_local void* t_stream = nullptr;
thread_local RecordedGraph* t_recording = nullptr;

struct IdleBlock {
    void* ptr;
    size_t bytes;
    void* stream;      // the stream whose work may still be using the block
    void* event;       // recorded on that stream at release; nullptr: nothing can be using it
};
struct DevicePool {
    std::mutex mu;
    std::multimap<size_t, IdleBlock> idle;
    int64_t device_allocs = 0, reused = 0, idle_bytes = 0;
};
DevicePool& pool_of(int32_t device)
{
    // never evicted, like the reference's device cache (cuda/gpu.rs:99-152), and never destroyed: buffers released while the
    // process winds down still find their pool
    static std::mutex* mu = new std::mutex();
    static std::map<int32_t, DevicePool*>* pools = new std::map<int32_t, DevicePool*>();
    std::lock_guard<std::mutex> lock(*mu);
    DevicePool*& p = (*pools)[device];
    if (!p) p = new DevicePool();
    return *p;
}
size_t pool_size_class(size_t bytes)
{
    if (bytes == 0) bytes = 1;
    const size_t unit = bytes <= (1u << 20) ? 512 : (64u << 10);      // little is wasted, and equal requests meet equal blocks
    return (bytes + unit - 1) / unit * unit;
}
// A block of at least `bytes`: from the pool when one is there that this thread's stream may touch, else from the device.
// *settled says whether nothing on the device can still be using the block (a host-side copy into it needs that).
int pool_alloc(int32_t device, size_t bytes, void** out, size_t* granted, bool* settled)
{
    const size_t want = pool_size_class(bytes);
    DevicePool& pool = pool_of(device);
    {
        std::lock_guard<std::mutex> lock(pool.mu);
        for (auto it = pool.idle.lower_bound(want); it != pool.idle.end() && it->first <= want + want / 4 + 4096; ++it) {
            IdleBlock& b = it->second;
            bool done = b.event == nullptr;
            if (!done && !t_recording) {      // (an event recorded into a graph cannot be asked; such blocks carry none)
                int32_t d = 0;
                if (incin_rocm_event_query(device, b.event, &d) == 0 && d) done = true;
            }
            if (!done && b.stream != t_stream) continue;
            if (b.event) incin_rocm_event_destroy(device, b.event);
            *out = b.ptr;
            *granted = b.bytes;
            *settled = done;
            pool.idle_bytes -= (int64_t)b.bytes;
            ++pool.reused;
            pool.idle.erase(it);
            return 0;
        }
    }
    if (t_recording) {
        // (no message from the C ABI for this one: the refusal is the pool's)
        return -1;
    }
    int rc = incin_rocm_alloc(device, want, out);
    if (rc == INCIN_ROCM_ENOMEM) {      // give back what is idle and try once more
        RocmBackend::trim_pool(device);
        rc = incin_rocm_alloc(device, want, out);
    }
    if (rc != 0) return rc;
    *granted = want;
    *settled = true;
    std::lock_guard<std::mutex> lock(pool.mu);
    ++pool.device_allocs;
    return 0;
}
void pool_release(int32_t device, void* ptr, size_t bytes)
{
    if (t_recording && t_recording->device == device) {      // the recorded kernels use it at every replay
        t_recording->retained.emplace_back(ptr, bytes);
        return;
    }
    IdleBlock b{ptr, bytes, t_stream, nullptr};
    if (incin_rocm_event_create(device, &b.event) != 0 || incin_rocm_event_record(device, b.event, t_stream) != 0) {
        // no event to be had: make sure nothing uses the block, then it needs none
        if (b.event) incin_rocm_event_destroy(device, b.event);
        b.event = nullptr;
        incin_rocm_sync(device);
    }
    DevicePool& pool = pool_of(device);
    std::lock_guard<std::mutex> lock(pool.mu);
    pool.idle_bytes += (int64_t)bytes;
    pool.idle.emplace(bytes, b);
}

std::vector<int64_t> contiguous_strides(const std::vector<int64_t>& shape)
{
    std::vector<int64_t> st(shape.size());
    int64_t acc = 1;
    for (int i = (int)shape.size() - 1; i >= 0; --i) {
        st[i] = acc;
        acc *= shape[i];
    }
    return st;
}

// A buffer of `bytes` (the pool may grant more).  *settled (may be null): nothing on the device can still be using it.
Error alloc_buffer(int32_t device, size_t bytes, std::shared_ptr<RocmBuffer>* out, bool* settled = nullptr)
{
    void* p = nullptr;
    size_t granted = 0;
    bool s = true;
    const int rc = pool_alloc(device, bytes, &p, &granted, &s);
    if (rc == -1)
        return err(ErrorKind::Msg, "ROCm allocation of " + std::to_string(bytes) + " bytes while a launch graph is being recorded: the pool holds no "
                                   "buffer of that size for this stream (run the recorded operators once before recording)");
    if (Error e = from_status(rc, device)) return e;
    if (settled) *settled = s;
    *out = std::make_shared<RocmBuffer>(device, p, granted);
    return ok();
}

Error alloc_storage(const std::vector<int64_t>& dims, DType dtype, int32_t device, RocmStorage* out, bool* settled = nullptr)
{
    int64_t n = 1;
    for (int64_t d : dims) {
        if (d < 0) return err(ErrorKind::ShapeMismatch, "negative extent in " + shape_str(dims));
        n *= d;
    }
    void* p = nullptr;
    const size_t bytes = (size_t)n * dtype_size(dtype);
    std::shared_ptr<RocmBuffer> buf;
    if (Error e = alloc_buffer(device, bytes, &buf, settled)) return e;
    p = buf->ptr();
    out->buffer = std::move(buf);
    out->shape = dims;
    out->strides = contiguous_strides(dims);
    out->offset_elements = 0;
    out->dtype = dtype;
    out->device = device;
    out->mask_tag.reset();
    return ok();
}

// strides of `s` seen through a right-aligned broadcast to `target` (rank >= s.rank); 0 where expanded
bool broadcast_strides(const std::vector<int64_t>& shape, const std::vector<int64_t>& strides,
                       const std::vector<int64_t>& target, std::vector<int64_t>* out)
{
    const size_t n = target.size(), r = shape.size();
    if (r > n) return false;
    out->assign(n, 0);
    for (size_t i = 0; i < r; ++i) {
        const size_t ti = n - r + i;
        if (shape[i] == target[ti]) (*out)[ti] = shape[i] == 1 ? 0 : strides[i];
        else if (shape[i] == 1) (*out)[ti] = 0;
        else return false;
    }
    return true;
}

}  // namespace

int64_t last_launch_count() { return g_launches; }

RocmBuffer::~RocmBuffer()
{
    if (ptr_) pool_release(device_, ptr_, bytes_);
}

RecordedGraph::~RecordedGraph()
{
    if (graph) incin_rocm_graph_destroy(device, graph);
    // (what the recording kept may be in use by a replay that is still running: release it like any other buffer, ordered
    // behind the calling thread's stream - the caller replays and destroys on one stream)
    for (auto& b : retained) pool_release(device, b.first, b.second);
}

void RocmBackend::set_stream(void* stream) { t_stream = stream; }
void* RocmBackend::stream() { return t_stream; }

Error RocmBackend::begin_recording(int32_t device)
{
    if (t_recording) return err(ErrorKind::Msg, "a launch graph is already being recorded on this thread");
    if (!t_stream) return err(ErrorKind::Msg, "recording needs a stream of its own (set_stream), not the default stream");
    if (Error e = from_status(incin_rocm_graph_begin(device, t_stream), device)) return e;
    t_recording = new RecordedGraph();
    t_recording->device = device;
    return ok();
}

Error RocmBackend::end_recording(std::unique_ptr<RecordedGraph>* out)
{
    if (!t_recording) return err(ErrorKind::Msg, "no launch graph is being recorded on this thread");
    std::unique_ptr<RecordedGraph> g(t_recording);
    t_recording = nullptr;
    if (Error e = from_status(incin_rocm_graph_end(g->device, t_stream, &g->graph), g->device)) return e;
    *out = std::move(g);
    return ok();
}

Error RocmBackend::replay(const RecordedGraph& g) { return from_status(incin_rocm_graph_launch(g.device, g.graph, t_stream), g.device); }

RocmBackend::PoolStats RocmBackend::pool_stats(int32_t device)
{
    DevicePool& pool = pool_of(device);
    std::lock_guard<std::mutex> lock(pool.mu);
    PoolStats s;
    s.device_allocs = pool.device_allocs;
    s.reused = pool.reused;
    s.idle_bytes = pool.idle_bytes;
    return s;
}

Error RocmBackend::trim_pool(int32_t device)
{
    if (Error e = from_status(incin_rocm_sync(device), device)) return e;
    DevicePool& pool = pool_of(device);
    std::lock_guard<std::mutex> lock(pool.mu);
    for (auto& kv : pool.idle) {
        if (kv.second.event) incin_rocm_event_destroy(device, kv.second.event);
        incin_rocm_free(device, kv.second.ptr);
    }
    pool.idle.clear();
    pool.idle_bytes = 0;
    return ok();
}

int64_t RocmStorage::numel() const
{
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
}

bool RocmStorage::is_contiguous() const
{
    int64_t acc = 1;
    for (int i = (int)shape.size() - 1; i >= 0; --i) {
        if (shape[i] != 1 && strides[i] != acc) return false;
        acc *= shape[i];
    }
    return true;
}

Error broadcast_shape(const std::vector<int64_t>& a, const std::vector<int64_t>& b, std::vector<int64_t>* out)
{
    const size_t n = std::max(a.size(), b.size());
    out->assign(n, 1);
    for (size_t i = 0; i < n; ++i) {
        const int64_t da = i + a.size() >= n ? a[i + a.size() - n] : 1;
        const int64_t db = i + b.size() >= n ? b[i + b.size() - n] : 1;
        if (da != db && da != 1 && db != 1)
            return err(ErrorKind::ShapeMismatch, "cannot broadcast shapes " + shape_str(a) + " and " + shape_str(b) +
                                                     ": incompatible at right-aligned axis " + std::to_string(i));
        (*out)[i] = std::max(da, db);
    }
    return ok();
}

Error RocmBackend::from_bytes(const void* bytes, size_t nbytes, const std::vector<int64_t>& dims, DType dtype, int32_t device,
                              RocmStorage* out)
{
    if ((int)dtype < 0 || (int)dtype > 2) return err(ErrorKind::UnsupportedDType, "dtype tag " + std::to_string((int)dtype) + " on backend Rocm");
    RocmStorage s;
    bool settled = true;
    if (Error e = alloc_storage(dims, dtype, device, &s, &settled)) return e;
    if ((size_t)s.numel() * dtype_size(dtype) != nbytes)
        return err(ErrorKind::Msg, "from_bytes: " + std::to_string(nbytes) + " bytes do not fill shape " + shape_str(dims));
    if (nbytes && !bytes) return err(ErrorKind::Msg, "from_bytes: null source");
    // (the copy does not go through the thread's stream: a block the pool handed over in stream order may still be read by
    // that stream's earlier work)
    if (!settled)
        if (Error e = from_status(t_stream ? incin_rocm_stream_sync(device, t_stream) : incin_rocm_sync(device), device)) return e;
    if (Error e = from_status(incin_rocm_memcpy_h2d(device, s.buffer->ptr(), bytes, nbytes), device)) return e;
    *out = std::move(s);
    return ok();
}

Error RocmBackend::to_bytes(const RocmStorage& s, std::vector<uint8_t>* out)
{
    const size_t isz = dtype_size(s.dtype);
    const int64_t n = s.numel();
    out->assign((size_t)n * isz, 0);
    if (n == 0) return ok();
    // (the synchronous point of the contract, cuda/backend.rs:2007-2045: the copies below go through the default stream,
    // which does not wait for a stream created here)
    if (t_stream)
        if (Error e = from_status(incin_rocm_stream_sync(s.device, t_stream), s.device)) return e;
    if (s.is_contiguous())
        return from_status(incin_rocm_memcpy_d2h(s.device, out->data(), s.data(), (size_t)n * isz), s.device);
    if (s.shape.size() <= 8) {          // strided or broadcast view: gather on the device, then one copy
        RocmStorage dense;
        if (Error e = contiguous(s, &dense)) return e;
        return from_status(incin_rocm_memcpy_d2h(s.device, out->data(), dense.data(), (size_t)n * isz), s.device);
    }
    // beyond the copy kernel's rank: fetch the whole allocation once, gather on the host
    std::vector<uint8_t> raw(s.buffer->bytes());
    if (Error e = from_status(incin_rocm_memcpy_d2h(s.device, raw.data(), s.buffer->ptr(), raw.size()), s.device)) return e;
    std::vector<int64_t> idx(s.shape.size(), 0);
    for (int64_t flat = 0; flat < n; ++flat) {
        int64_t off = s.offset_elements;
        for (size_t a = 0; a < idx.size(); ++a) off += idx[a] * s.strides[a];
        std::memcpy(out->data() + (size_t)flat * isz, raw.data() + (size_t)off * isz, isz);
        for (int a = (int)idx.size() - 1; a >= 0; --a) {
            if (++idx[a] < s.shape[a]) break;
            idx[a] = 0;
        }
    }
    return ok();
}

// CpuStorage::contiguous (cpu/storage.rs:407-440): a fresh dense copy of a view, here gathered by one kernel.
Error RocmBackend::contiguous(const RocmStorage& s, RocmStorage* out)
{
    if (s.is_contiguous()) {
        *out = s;
        return ok();
    }
    if (s.shape.size() > 8) return err(ErrorKind::UnsupportedBackendOperation, "contiguous: rank above 8 on backend Rocm");
    RocmStorage dense;
    if (Error e = alloc_storage(s.shape, s.dtype, s.device, &dense)) return e;
    if (dense.numel() > 0) {
        if (Error e = from_status(incin_rocm_copy_strided(s.device, dense.buffer->ptr(), s.data(), (int32_t)s.shape.size(), s.shape.data(),
                                                          s.strides.data(), (int32_t)dtype_size(s.dtype), t_stream), s.device))
            return e;
    }
    *out = std::move(dense);
    return ok();
}

// An operand of attention whose last axis is strided (a transposed view, cpu/storage.rs:308-325), made dense along its
// last axes.  Axes the view only repeats (stride 0) are not expanded: they are copied at extent 1 and stay broadcast.
static Error dense_last_axis(const RocmStorage& s, RocmStorage* out)
{
    // (the last axis is the one the copy is for: a view that repeats one element along it - broadcast_as of [.., S, 1] -
    // is written out at its full extent)
    const size_t last = s.shape.size() - 1;
    RocmStorage squeezed = s;
    for (size_t a = 0; a < last; ++a)
        if (s.strides[a] == 0) squeezed.shape[a] = std::min<int64_t>(s.shape[a], 1);
    RocmStorage dense;
    if (Error e = RocmBackend::contiguous(squeezed, &dense)) return e;
    for (size_t a = 0; a < last; ++a)
        if (s.strides[a] == 0) { dense.shape[a] = s.shape[a]; dense.strides[a] = 0; }
    if (dense.strides[last] != 1 && dense.shape[last] > 1)
        return err(ErrorKind::UnsupportedBackendOperation, "scaled_dot_product_attention: could not make the last axis of " +
                                                               shape_str(s.shape) + " dense on backend Rocm");
    dense.mask_tag.reset();
    *out = std::move(dense);
    return ok();
}

// The gradient of an operand that was broadcast to `g`'s shape, summed back to the operand's shape `target`
// (right-aligned; cpu/tape.rs:243-265): leading axes the operand does not have and axes where it has extent 1 are summed
// away.  `g` is dense.
static Error sum_to_shape(const RocmStorage& g, const std::vector<int64_t>& target, RocmStorage* out)
{
    const int r = (int)g.shape.size(), pad = r - (int)target.size();
    if (pad < 0 || r > 8) return err(ErrorKind::UnsupportedBackendOperation, "unbroadcast: rank above 8 on backend Rocm");
    std::vector<int64_t> kept(r, 1);
    for (int a = pad; a < r; ++a) {
        if (target[a - pad] != g.shape[a] && target[a - pad] != 1)
            return err(ErrorKind::ShapeMismatch, "unbroadcast: " + shape_str(g.shape) + " does not reduce to " + shape_str(target));
        kept[a] = target[a - pad];
    }
    RocmStorage dst;
    if (Error e = alloc_storage(target, g.dtype, g.device, &dst)) return e;
    if (Error e = from_status(incin_rocm_sum_to_shape(g.device, (int32_t)g.dtype, dst.buffer->ptr(), g.data(), r, g.shape.data(), kept.data(), t_stream), g.device))
        return e;
    *out = std::move(dst);
    return ok();
}

Error RocmBackend::transpose(const RocmStorage& s, int a, int b, RocmStorage* out)
{
    const int r = (int)s.shape.size();
    if (a < 0 || b < 0 || a >= r || b >= r) return err(ErrorKind::ShapeMismatch, "transpose: axis out of range for rank " + std::to_string(r));
    *out = s;
    std::swap(out->shape[a], out->shape[b]);
    std::swap(out->strides[a], out->strides[b]);
    out->mask_tag.reset();
    return ok();
}

Error RocmBackend::broadcast_as(const RocmStorage& s, const std::vector<int64_t>& dims, RocmStorage* out)
{
    std::vector<int64_t> st;
    if (!broadcast_strides(s.shape, s.strides, dims, &st))
        return err(ErrorKind::ShapeMismatch, "cannot broadcast " + shape_str(s.shape) + " to " + shape_str(dims));
    *out = s;
    out->shape = dims;
    out->strides = st;
    out->mask_tag.reset();
    return ok();
}

Error RocmBackend::narrow(const RocmStorage& s, int dim, int64_t start, int64_t len, RocmStorage* out)
{
    const int r = (int)s.shape.size();
    if (dim < 0 || dim >= r || start < 0 || len < 0 || start + len > s.shape[dim])
        return err(ErrorKind::ShapeMismatch, "narrow: range out of bounds for " + shape_str(s.shape));
    *out = s;
    out->shape[dim] = len;
    out->offset_elements += start * s.strides[dim];
    out->mask_tag.reset();
    return ok();
}

Error RocmBackend::reshape(const RocmStorage& s, const std::vector<int64_t>& dims, RocmStorage* out)
{
    int64_t n = 1;
    for (int64_t d : dims) {
        if (d < 0) return err(ErrorKind::ShapeMismatch, "reshape: negative extent in " + shape_str(dims));
        n *= d;
    }
    if (n != s.numel())
        return err(ErrorKind::ShapeMismatch, "reshape: " + shape_str(s.shape) + " has " + std::to_string(s.numel()) +
                                                 " elements, " + shape_str(dims) + " has " + std::to_string(n));
    RocmStorage dense;                  // a view that is not dense is materialised first, as the reference's reshape does
    if (Error e = contiguous(s, &dense)) return e;
    *out = dense;
    out->shape = dims;
    out->strides.assign(dims.size(), 1);
    for (int i = (int)dims.size() - 2; i >= 0; --i) out->strides[i] = out->strides[i + 1] * dims[i + 1];
    out->mask_tag.reset();
    return ok();
}

Error RocmBackend::upload_i32(const std::vector<int32_t>& values, int32_t device, std::shared_ptr<RocmBuffer>* out)
{
    const size_t bytes = values.size() * sizeof(int32_t);
    std::shared_ptr<RocmBuffer> buf;
    bool settled = true;
    if (Error e = alloc_buffer(device, bytes ? bytes : 4, &buf, &settled)) return e;
    if (bytes) {
        if (!settled)      // (a host-side copy into a block that earlier work of the stream may still read)
            if (Error e = from_status(t_stream ? incin_rocm_stream_sync(device, t_stream) : incin_rocm_sync(device), device)) return e;
        if (Error e = from_status(incin_rocm_memcpy_h2d(device, buf->ptr(), values.data(), bytes), device)) return e;
    }
    *out = std::move(buf);
    return ok();
}

Error RocmBackend::tag_causal(const RocmStorage& mask, RocmStorage* out)
{
    if (mask.shape.size() < 2) return err(ErrorKind::ShapeMismatch, "a causal mask has at least two axes");
    *out = mask;
    out->mask_tag = MaskTag{MaskTag::Causal, nullptr, 0};
    return ok();
}

Error RocmBackend::tag_key_padding(const RocmStorage& mask, const std::vector<int32_t>& lens, RocmStorage* out)
{
    std::shared_ptr<RocmBuffer> buf;
    if (Error e = upload_i32(lens, mask.device, &buf)) return e;
    *out = mask;
    out->mask_tag = MaskTag{MaskTag::KeyPadding, buf, (int64_t)lens.size()};
    return ok();
}

Error RocmBackend::infer_mask_tag(const RocmStorage& mask, RocmStorage* out, int* kind)
{
    *out = mask;
    if (kind) *kind = 0;
    const size_t r = mask.shape.size();
    if (r < 2 || r > 4 || mask.mask_tag) return ok();
    // [A0, A1, rows, Skv]: missing leading axes are 1
    int64_t shape[4] = {1, 1, 1, 1}, strides[4] = {0, 0, 0, 0};
    for (size_t a = 0; a < r; ++a) {
        shape[4 - r + a] = mask.shape[a];
        strides[4 - r + a] = mask.shape[a] == 1 ? 0 : mask.strides[a];
    }
    const int64_t A0 = shape[0], A1 = shape[1], R = shape[2], Skv = shape[3];
    const int64_t n = A0 * A1 * R;
    if (n <= 0 || Skv <= 0 || n > (1 << 26)) return ok();
    std::shared_ptr<RocmBuffer> lims_dev;
    if (Error e = alloc_buffer(mask.device, (size_t)n * sizeof(int32_t), &lims_dev)) return e;
    if (Error e = from_status(incin_rocm_mask_row_limits(mask.device, (int32_t)mask.dtype, mask.data(), shape, strides,
                                                         static_cast<int32_t*>(lims_dev->ptr()), t_stream), mask.device))
        return e;
    if (Error e = from_status(t_stream ? incin_rocm_stream_sync(mask.device, t_stream) : incin_rocm_sync(mask.device), mask.device)) return e;
    std::vector<int32_t> lims((size_t)n);
    if (Error e = from_status(incin_rocm_memcpy_d2h(mask.device, lims.data(), lims_dev->ptr(), (size_t)n * sizeof(int32_t)), mask.device)) return e;
    // per index of the first axis: the count the last row states; then: are all rows that count (key padding), or the smaller
    // of it and the causal limit of the row (both; without a count below Skv: causal)?
    std::vector<int32_t> counts((size_t)A0);
    bool plain = true, causal = R > 1;
    for (int64_t a0 = 0; a0 < A0; ++a0) {
        const int32_t L = lims[(size_t)((a0 * A1) * R + (R - 1))];
        counts[(size_t)a0] = L;
        for (int64_t a1 = 0; a1 < A1; ++a1)
            for (int64_t i = 0; i < R; ++i) {
                const int32_t lm = lims[(size_t)((a0 * A1 + a1) * R + i)];
                if (lm < 0) return ok();
                const int64_t c = std::min<int64_t>(std::max<int64_t>(i + 1 + Skv - R, 0), Skv);
                plain = plain && lm == L;
                causal = causal && lm == std::min<int64_t>(c, L);
            }
    }
    if (!plain && !causal) return ok();
    bool padded = false;
    for (int32_t c : counts) padded = padded || c < Skv;
    if (!padded) {
        if (!causal) return ok();               // all zeros: the mask says nothing, and costs nothing that matters as it is
        out->mask_tag = MaskTag{MaskTag::Causal, nullptr, 0};
        if (kind) *kind = 1;
        return ok();
    }
    // key counts go by batch entry: only a rank-4 mask with more than one entry on its first axis says which rows of the
    // scores belong to which (under the operator's right-aligned broadcast a shorter mask's first axis is the head axis,
    // and a single entry may be repeated over a batch whose size the mask does not know)
    if (r != 4 || A0 == 1) return ok();
    std::shared_ptr<RocmBuffer> buf;
    if (Error e = upload_i32(counts, mask.device, &buf)) return e;
    out->mask_tag = MaskTag{plain ? MaskTag::KeyPadding : MaskTag::CausalKeyPadding, buf, (int64_t)counts.size()};
    if (kind) *kind = plain ? 2 : 3;
    return ok();
}

Error RocmBackend::scaled_dot_product_attention(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v,
                                                const RocmStorage* mask, std::optional<double> scale, RocmStorage* out)
{
    return attention(q, k, v, mask, scale, MaskFacts{}, out);
}

Error RocmBackend::attention(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                             std::optional<double> scale, const MaskFacts& facts, RocmStorage* out)
{
    return attention_impl(q, k, v, mask, scale, facts, nullptr, out, nullptr);
}

Error RocmBackend::attention_backward(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                                      std::optional<double> scale, const MaskFacts& facts, const RocmStorage& grad_out,
                                      RocmStorage* out, AttentionGrads* grads)
{
    return attention_impl(q, k, v, mask, scale, facts, &grad_out, out, grads);
}

// Forward, and with `grads` the backward after it: every launch of the forward keeps its row normalisers, and
// incin_rocm_sdpa_bwd turns them, the output and the upstream gradient into dq, dk, dv of that launch's slice.
Error RocmBackend::attention_impl(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                                  std::optional<double> scale, const MaskFacts& facts, const RocmStorage* grad_out,
                                  RocmStorage* out, AttentionGrads* grads)
{
    static const char* OP = "scaled_dot_product_attention";
    // -- devices and dtypes, in the order the reference's checks fire ------------------------------------
    if (q.device != k.device || q.device != v.device || (mask && mask->device != q.device))
        return err(ErrorKind::DeviceMismatch, std::string(OP) + ": operands live on different devices");
    if (k.dtype != q.dtype || v.dtype != q.dtype || (mask && mask->dtype != q.dtype))
        return err(ErrorKind::DTypeStorageMismatch, std::string(OP) + ": operands have different dtypes");
    // -- shapes (cpu/ops/matmul.rs:170-196) ------------------------------------------------------------
    const int qr = (int)q.shape.size(), kr = (int)k.shape.size(), vr = (int)v.shape.size();
    if (qr < 2 || kr < 2 || vr < 2)
        return err(ErrorKind::ShapeMismatch, std::string(OP) + ": operands need rank >= 2; got q " + shape_str(q.shape) +
                                                 ", k " + shape_str(k.shape) + ", v " + shape_str(v.shape));
    const int64_t Sq = q.shape[qr - 2], D = q.shape[qr - 1], Skv = k.shape[kr - 2], Dv = v.shape[vr - 1];
    if (k.shape[kr - 1] != D)
        return err(ErrorKind::ShapeMismatch, std::string(OP) + ": q and k inner dims must match: q " + shape_str(q.shape) + ", k " + shape_str(k.shape));
    if (v.shape[vr - 2] != Skv)
        return err(ErrorKind::ShapeMismatch, std::string(OP) + ": k and v key counts must match: k " + shape_str(k.shape) + ", v " + shape_str(v.shape));
    // The kernels read rows of unit stride.  The reference takes any view (cpu/storage.rs:308-325; k = transpose of
    // [.., D, Skv] storage is pinned at cpu/ops/matmul.rs:677-724): such an operand is gathered into a dense temporary
    // first, as CpuStorage::contiguous would, and the operator runs on that.
    {
        const bool fq = q.strides[qr - 1] != 1 && D > 1, fk = k.strides[kr - 1] != 1 && D > 1, fv = v.strides[vr - 1] != 1 && Dv > 1;
        if (fq || fk || fv) {
            if (qr > 8 || kr > 8 || vr > 8)
                return err(ErrorKind::UnsupportedBackendOperation, std::string(OP) + ": a strided last axis needs rank <= 8 on backend Rocm");
            RocmStorage qd = q, kd = k, vd = v;
            if (fq) if (Error e = dense_last_axis(q, &qd)) return e;
            if (fk) if (Error e = dense_last_axis(k, &kd)) return e;
            if (fv) if (Error e = dense_last_axis(v, &vd)) return e;
            // (the temporaries are released in stream order when this returns: nothing to wait for)
            return attention_impl(qd, kd, vd, mask, scale, facts, grad_out, out, grads);
        }
    }

    // -- gradients of a view that repeats its storage along a batch axis (stride 0 at an extent above 1): to the reference
    // such an operand has the view's shape and every repeated slice gets a gradient of its own (cpu/tape.rs:243-246: no
    // sum where the shapes agree), so the view is written out and treated like any dense operand.
    if (grads) {
        auto repeats = [](const RocmStorage& x) {
            for (size_t a = 0; a + 2 < x.shape.size(); ++a)
                if (x.shape[a] > 1 && x.strides[a] == 0) return true;
            return false;
        };
        if (repeats(q) || repeats(k) || repeats(v)) {
            RocmStorage qd = q, kd = k, vd = v;
            if (repeats(q)) if (Error e = contiguous(q, &qd)) return e;
            if (repeats(k)) if (Error e = contiguous(k, &kd)) return e;
            if (repeats(v)) if (Error e = contiguous(v, &vd)) return e;
            return attention_impl(qd, kd, vd, mask, scale, facts, grad_out, out, grads);
        }
    }

    // -- a mask that adds query rows: scores [.., 1, Skv] + mask [.., R, Skv] is [.., R, Skv] in the reference (its add
    // broadcasts both ways, cpu/ops/shape_ops.rs:1262-1266 with cpu/stride.rs:86-106): q's one row is repeated R times
    // (a stride-0 view, written out so that every kernel sees rows of its own), and a gradient sums the rows back.
    if (mask && mask->shape.size() >= 2 && Sq == 1) {
        const int64_t mrows = mask->shape[mask->shape.size() - 2];
        if (mrows > 1) {
            std::vector<int64_t> dims = q.shape;
            dims[qr - 2] = mrows;
            RocmStorage qv, qd;
            if (Error e = broadcast_as(q, dims, &qv)) return e;
            if (Error e = contiguous(qv, &qd)) return e;
            if (!grads) return attention_impl(qd, k, v, mask, scale, facts, grad_out, out, grads);
            AttentionGrads g2;
            if (Error e = attention_impl(qd, k, v, mask, scale, facts, grad_out, out, &g2)) return e;
            if (Error e = sum_to_shape(g2.dq, q.shape, &grads->dq)) return e;
            grads->dk = std::move(g2.dk);
            grads->dv = std::move(g2.dv);
            return ok();
        }
    }

    // -- batch axes: broadcast(broadcast(broadcast(q, k), mask), v), NumPy rule (cpu/ops/matmul.rs:198-221 for the two
    // products, cpu/stride.rs:86-106 for the mask's add, which may add leading axes or widen axes of extent 1) ------------
    const std::vector<int64_t> qb(q.shape.begin(), q.shape.end() - 2), kb(k.shape.begin(), k.shape.end() - 2),
        vb(v.shape.begin(), v.shape.end() - 2);
    std::vector<int64_t> bshape, tmp;
    if (Error e = broadcast_shape(qb, kb, &tmp)) return e;
    std::vector<int64_t> mshape, mstr;
    if (mask) {
        mshape = mask->shape;
        mstr = mask->strides;
        while ((int)mshape.size() < 2) {
            mshape.insert(mshape.begin(), 1);
            mstr.insert(mstr.begin(), 0);
        }
        const int64_t mr = mshape[mshape.size() - 2], mc = mshape[mshape.size() - 1];
        std::vector<int64_t> full = tmp;
        full.push_back(Sq);
        full.push_back(Skv);
        // (a mask with more keys than k has would widen the scores past v's rows: the second product refuses that)
        if ((mr != 1 && mr != Sq) || (mc != 1 && mc != Skv))
            return err(ErrorKind::ShapeMismatch, std::string(OP) + ": mask " + shape_str(mask->shape) +
                                                     " does not broadcast to the scores " + shape_str(full));
        std::vector<int64_t> tmp2;
        if (broadcast_shape(tmp, std::vector<int64_t>(mshape.begin(), mshape.end() - 2), &tmp2))
            return err(ErrorKind::ShapeMismatch, std::string(OP) + ": mask " + shape_str(mask->shape) +
                                                     " does not broadcast to the scores " + shape_str(full));
        tmp = tmp2;
    }
    if (Error e = broadcast_shape(tmp, vb, &bshape)) return e;
    const int nb = (int)bshape.size();
    std::vector<int64_t> qs, ks, vs, ms;
    broadcast_strides(qb, std::vector<int64_t>(q.strides.begin(), q.strides.end() - 2), bshape, &qs);
    broadcast_strides(kb, std::vector<int64_t>(k.strides.begin(), k.strides.end() - 2), bshape, &ks);
    broadcast_strides(vb, std::vector<int64_t>(v.strides.begin(), v.strides.end() - 2), bshape, &vs);

    // -- mask: None | tagged | dense additive, seen through the broadcast to [..b, Sq, Skv] ---------------------------
    int64_t m_si = 0, m_sj = 0;
    bool dense_mask = false;
    if (mask) {
        std::vector<int64_t> full = bshape;
        full.push_back(Sq);
        full.push_back(Skv);
        std::vector<int64_t> mfull;
        if (!broadcast_strides(mshape, mstr, full, &mfull))
            return err(ErrorKind::ShapeMismatch, std::string(OP) + ": mask " + shape_str(mask->shape) +
                                                     " does not broadcast to the scores " + shape_str(full));
        if (!mask->mask_tag) {
            dense_mask = true;
            ms.assign(mfull.begin(), mfull.end() - 2);
            m_si = mfull[nb];
            m_sj = mfull[nb + 1];
        }
    }

    // -- output: fresh contiguous [..b, Sq, Dv] of the input dtype -----------------------------------------------
    std::vector<int64_t> oshape = bshape;
    oshape.push_back(Sq);
    oshape.push_back(Dv);
    RocmStorage o;
    if (Error e = alloc_storage(oshape, q.dtype, q.device, &o)) return e;
    const std::vector<int64_t> os(o.strides.begin(), o.strides.end() - 2);

    // -- gradients: dense storages over the batch axes the launches run over; an operand repeated along a batch axis gets its
    // gradient summed over that axis afterwards (cpu/tape.rs:243-265) - except keys and values shared by a group of query
    // heads, which the kernels sum themselves (the group axis is found below: the storages are laid out after it) -----------
    RocmStorage gq, gk, gv, grad_dense;
    std::vector<int64_t> gqs, gks, gvs;
    if (grads) {
        if (!grad_out || grad_out->device != q.device) return err(ErrorKind::DeviceMismatch, std::string(OP) + " backward: the upstream gradient lives on another device");
        if (grad_out->dtype != q.dtype) return err(ErrorKind::DTypeStorageMismatch, std::string(OP) + " backward: the upstream gradient has another dtype");
        if (grad_out->shape != oshape)
            return err(ErrorKind::ShapeMismatch, std::string(OP) + " backward: upstream gradient " + shape_str(grad_out->shape) + ", output " + shape_str(oshape));
        // the kernels read the upstream gradient with the output's strides: any other view is gathered first
        if (Error e = contiguous(*grad_out, &grad_dense)) return e;
        grad_out = &grad_dense;
    }

    // -- collapse the batch axes into (outer..., B, Hkv, G) ----------------------------------------------------
    // G: the last batch axis when k and v are broadcast along it and q is not (the reference's way to write
    // grouped-query attention: q [.., Hkv, G, S, D] against k, v [.., Hkv, 1, S, D]); Hkv: the axis before it;
    // B: the one before that; anything further left is looped over here, one launch per index.
    int g_ax = -1, h_ax = -1, b_ax = -1;
    int next = nb - 1;
    if (next >= 0 && bshape[next] > 1 && ks[next] == 0 && vs[next] == 0 && qs[next] != 0) g_ax = next--;
    // rank-4 operands read [B, H, S, D] (k, v broadcast over H: one shared kv head); rank-5 and up read
    // [.., B, Hkv, G, S, D]
    if (next >= 0 && !(g_ax >= 0 && next == 0)) h_ax = next--;
    if (next >= 0) b_ax = next--;
    const int n_outer = next + 1;
    bool sum_q = false, sum_k = false, sum_v = false;      // a gradient storage is wider than its operand
    if (grads) {
        // shape of an operand's gradient as the launches write it: the batch shape, with extent 1 kept only on the group axis
        // of k and v
        auto launch_shape = [&](const RocmStorage& x, bool kv, bool* wider) {
            std::vector<int64_t> dims(bshape);
            const int pad = nb - ((int)x.shape.size() - 2);
            for (int a = 0; a < nb; ++a) {
                const int64_t own = a >= pad ? x.shape[a - pad] : 1;
                if (kv && a == g_ax) dims[a] = 1;
                else if (own != bshape[a]) *wider = true;
            }
            dims.push_back(x.shape[x.shape.size() - 2]);
            dims.push_back(x.shape[x.shape.size() - 1]);
            return dims;
        };
        const std::vector<int64_t> gq_dims = launch_shape(q, false, &sum_q), gk_dims = launch_shape(k, true, &sum_k),
                                   gv_dims = launch_shape(v, true, &sum_v);
        if (nb + 2 > 8 && (sum_q || sum_k || sum_v))
            return err(ErrorKind::UnsupportedBackendOperation, std::string(OP) + " backward: summing the gradient of a broadcast operand needs rank <= 8 on backend Rocm");
        if (Error e = alloc_storage(gq_dims, q.dtype, q.device, &gq)) return e;
        if (Error e = alloc_storage(gk_dims, k.dtype, k.device, &gk)) return e;
        if (Error e = alloc_storage(gv_dims, v.dtype, v.device, &gv)) return e;
        broadcast_strides(std::vector<int64_t>(gq_dims.begin(), gq_dims.end() - 2), std::vector<int64_t>(gq.strides.begin(), gq.strides.end() - 2), bshape, &gqs);
        broadcast_strides(std::vector<int64_t>(gk_dims.begin(), gk_dims.end() - 2), std::vector<int64_t>(gk.strides.begin(), gk.strides.end() - 2), bshape, &gks);
        broadcast_strides(std::vector<int64_t>(gv_dims.begin(), gv_dims.end() - 2), std::vector<int64_t>(gv.strides.begin(), gv.strides.end() - 2), bshape, &gvs);
    }
    int64_t G = g_ax >= 0 ? bshape[g_ax] : 1;
    int64_t Hkv = h_ax >= 0 ? bshape[h_ax] : 1;
    const int64_t B = b_ax >= 0 ? bshape[b_ax] : 1;
    // query head hq = hkv * G + g must be one stride for q, o and the mask
    bool fold_g = g_ax >= 0 && h_ax >= 0;
    if (fold_g) {
        const bool q_ok = qs[h_ax] == G * qs[g_ax] || Hkv == 1;
        const bool o_ok = os[h_ax] == G * os[g_ax] || Hkv == 1;
        const bool m_ok = !dense_mask || (ms[h_ax] == G * ms[g_ax]) || Hkv == 1;
        if (!(q_ok && o_ok && m_ok)) fold_g = false;
    }
    // when the group axis cannot be folded into the head axis, the kv-head axis joins the outer loop
    std::vector<int> outer_axes;
    for (int a = 0; a < n_outer; ++a) outer_axes.push_back(a);
    int head_ax = h_ax;       // axis whose stride is the head stride of q / o / mask
    int64_t Hq = Hkv * G, Hkv_launch = Hkv;
    if (g_ax >= 0 && !fold_g) {
        if (h_ax >= 0) outer_axes.push_back(h_ax);
        head_ax = g_ax;
        Hq = G;
        Hkv_launch = 1;
    } else if (g_ax >= 0) {
        head_ax = g_ax;       // stride of one query head is the stride of the group axis
    }

    const double s64 = scale ? *scale : 1.0 / std::sqrt((double)D);       // shape_ops.rs:1259-1260 (q's last dim)
    incin_rocm_sdpa_desc_t d;
    std::memset(&d, 0, sizeof(d));
    d.dtype = (int32_t)q.dtype;
    d.device = q.device;
    d.B = B; d.Hq = Hq; d.Hkv = Hkv_launch; d.Sq = Sq; d.Skv = Skv; d.D = D; d.Dv = Dv;
    auto st = [&](const std::vector<int64_t>& s, int ax) { return ax >= 0 ? s[ax] : 0; };
    d.q_stride[0] = st(qs, b_ax); d.q_stride[1] = st(qs, head_ax); d.q_stride[2] = q.strides[qr - 2];
    d.o_stride[0] = st(os, b_ax); d.o_stride[1] = st(os, head_ax); d.o_stride[2] = o.strides[nb];
    // k, v: one stride per kv head (the axis before the group axis, or the head axis itself when there is no group)
    const int kv_head_ax = (g_ax >= 0) ? (fold_g ? h_ax : -1) : h_ax;
    d.k_stride[0] = st(ks, b_ax); d.k_stride[1] = st(ks, kv_head_ax); d.k_stride[2] = k.strides[kr - 2];
    d.v_stride[0] = st(vs, b_ax); d.v_stride[1] = st(vs, kv_head_ax); d.v_stride[2] = v.strides[vr - 2];
    d.scale = (float)s64;                                                   // elementwise_kernel.rs:87
    if (mask && mask->mask_tag) {
        if (mask->mask_tag->kind != MaskTag::KeyPadding) d.causal = 1;
        if (mask->mask_tag->kind != MaskTag::Causal) {
            if (mask->mask_tag->lens_count != B || n_outer != 0 || (g_ax >= 0 && !fold_g && h_ax >= 0))
                return err(ErrorKind::ShapeMismatch, std::string(OP) + ": key-padding lengths must have one entry per batch index");
            d.kv_lens = static_cast<const int32_t*>(mask->mask_tag->lens->ptr());
        }
    } else if (dense_mask) {
        d.mask_stride[0] = st(ms, b_ax); d.mask_stride[1] = st(ms, head_ax); d.mask_stride[2] = m_si; d.mask_stride[3] = m_sj;
    }

    // facts stated by the caller's descriptor rather than by a mask storage; they combine with either kind of mask
    if (facts.causal) d.causal = 1;
    if (facts.kv_lens) {
        if (d.kv_lens) return err(ErrorKind::ShapeMismatch, std::string(OP) + ": key lengths given twice (descriptor and mask tag)");
        if (facts.kv_lens_count != B || n_outer != 0 || (g_ax >= 0 && !fold_g && h_ax >= 0))
            return err(ErrorKind::ShapeMismatch, std::string(OP) + ": key-padding lengths must have one entry per batch index");
        d.kv_lens = static_cast<const int32_t*>(facts.kv_lens->ptr());
    }
    if (facts.q_lens) {
        if (facts.q_lens_count != B || n_outer != 0 || (g_ax >= 0 && !fold_g && h_ax >= 0))
            return err(ErrorKind::ShapeMismatch, std::string(OP) + ": query lengths must have one entry per batch index");
        d.q_lens = static_cast<const int32_t*>(facts.q_lens->ptr());
    }

    const size_t isz = dtype_size(q.dtype);
    // iterate the outer axes
    std::vector<int64_t> oidx(outer_axes.size(), 0);
    int64_t n_launch = 1;
    for (int a : outer_axes) n_launch *= bshape[a];
    std::shared_ptr<RocmBuffer> workspace, bwd_workspace, lse;
    g_launches = 0;
    for (int64_t it = 0; it < n_launch; ++it) {
        int64_t qo = q.offset_elements, ko = k.offset_elements, vo = v.offset_elements, oo = 0, mo = mask ? mask->offset_elements : 0;
        for (size_t a = 0; a < outer_axes.size(); ++a) {
            const int ax = outer_axes[a];
            qo += oidx[a] * qs[ax]; ko += oidx[a] * ks[ax]; vo += oidx[a] * vs[ax]; oo += oidx[a] * os[ax];
            if (dense_mask) mo += oidx[a] * ms[ax];
        }
        d.q = static_cast<const char*>(q.buffer->ptr()) + qo * (int64_t)isz;
        d.k = static_cast<const char*>(k.buffer->ptr()) + ko * (int64_t)isz;
        d.v = static_cast<const char*>(v.buffer->ptr()) + vo * (int64_t)isz;
        d.o = static_cast<char*>(o.buffer->ptr()) + oo * (int64_t)isz;
        d.add_mask = dense_mask ? static_cast<const char*>(mask->buffer->ptr()) + mo * (int64_t)isz : nullptr;
        if (grads) {
            if (!lse) {
                const size_t lbytes = (size_t)std::max<int64_t>(B * Hq * Sq, 1) * sizeof(float);
                if (Error e = alloc_buffer(q.device, lbytes, &lse)) return e;
            }
            d.lse = static_cast<float*>(lse->ptr());
        }
        size_t ws_bytes = 0;
        int32_t splits = 0;
        d.workspace = nullptr;
        d.workspace_bytes = 0;
        if (Error e = from_status(incin_rocm_sdpa_workspace(&d, &ws_bytes, &splits, nullptr), q.device)) return e;
        if (ws_bytes) {
            if (!workspace || workspace->bytes() < ws_bytes)
                if (Error e = alloc_buffer(q.device, ws_bytes, &workspace)) return e;
            d.workspace = workspace->ptr();
            d.workspace_bytes = workspace->bytes();
        }
        if (Error e = from_status(incin_rocm_sdpa_fwd(&d, t_stream), q.device)) return e;
        ++g_launches;
        if (grads) {
            int64_t gqo = 0, gko = 0, gvo = 0;
            for (size_t a = 0; a < outer_axes.size(); ++a) {
                const int ax = outer_axes[a];
                gqo += oidx[a] * gqs[ax]; gko += oidx[a] * gks[ax]; gvo += oidx[a] * gvs[ax];
            }
            incin_rocm_sdpa_bwd_desc_t bd;
            std::memset(&bd, 0, sizeof(bd));
            bd.fwd = d;
            bd.fwd.workspace = nullptr;
            bd.fwd.workspace_bytes = 0;
            bd.d_o = static_cast<const char*>(grad_out->data()) + oo * (int64_t)isz;
            bd.d_q = static_cast<char*>(gq.buffer->ptr()) + gqo * (int64_t)isz;
            bd.d_k = static_cast<char*>(gk.buffer->ptr()) + gko * (int64_t)isz;
            bd.d_v = static_cast<char*>(gv.buffer->ptr()) + gvo * (int64_t)isz;
            for (int a = 0; a < 3; ++a) bd.d_o_stride[a] = d.o_stride[a];
            bd.d_q_stride[0] = st(gqs, b_ax); bd.d_q_stride[1] = st(gqs, head_ax); bd.d_q_stride[2] = D;
            bd.d_k_stride[0] = st(gks, b_ax); bd.d_k_stride[1] = st(gks, kv_head_ax); bd.d_k_stride[2] = D;
            bd.d_v_stride[0] = st(gvs, b_ax); bd.d_v_stride[1] = st(gvs, kv_head_ax); bd.d_v_stride[2] = Dv;
            size_t bws = 0;
            if (Error e = from_status(incin_rocm_sdpa_bwd_workspace(&bd, &bws), q.device)) return e;
            if (bws) {
                if (!bwd_workspace || bwd_workspace->bytes() < bws)
                    if (Error e = alloc_buffer(q.device, bws, &bwd_workspace)) return e;
                bd.workspace = bwd_workspace->ptr();
                bd.workspace_bytes = bwd_workspace->bytes();
            }
            if (Error e = from_status(incin_rocm_sdpa_bwd(&bd, t_stream), q.device)) return e;
        }
        for (int a = (int)oidx.size() - 1; a >= 0; --a) {
            if (++oidx[a] < bshape[outer_axes[a]]) break;
            oidx[a] = 0;
        }
    }
    // (the workspaces and the row normalisers are still in use by the launches above: they are released in stream order)
    *out = std::move(o);
    if (grads) {
        // (a gradient storage of the operand's own extents only needs the operand's rank back)
        auto finish = [&](RocmStorage& g, const RocmStorage& x, bool wider, RocmStorage* dst) -> Error {
            if (wider) return sum_to_shape(g, x.shape, dst);
            g.shape = x.shape;
            g.strides = contiguous_strides(x.shape);
            *dst = std::move(g);
            return ok();
        };
        if (Error e = finish(gq, q, sum_q, &grads->dq)) return e;
        if (Error e = finish(gk, k, sum_k, &grads->dk)) return e;
        if (Error e = finish(gv, v, sum_v, &grads->dv)) return e;
    }
    return ok();
}

}  // namespace incin_rocm_host
