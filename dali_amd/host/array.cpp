// Array handles, buffer views, memory placement and the op:: factories.
#include <algorithm>
#include <limits>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <numeric>

#include "../../include/dali_hip.h"
#include "expr.h"

namespace dali {

int size_of_dtype(DType dtype) { return dtype == DTYPE_DOUBLE ? 8 : 4; }

std::string dtype_to_cpp_name(DType dtype) {
    switch (dtype) {
        case DTYPE_FLOAT: return "float";
        case DTYPE_DOUBLE: return "double";
        default: return "int";
    }
}

std::string shape_str(const std::vector<int>& shape) {
    std::ostringstream ss;
    ss << "[";
    for (size_t i = 0; i < shape.size(); ++i) ss << (i ? ", " : "") << shape[i];
    ss << "]";
    return ss.str();
}

void check_hip(int status, const char* what) {
    if (status != 0) throw std::runtime_error(make_message(what, ": ", dali_hip_last_error()));
}

std::vector<int> contiguous_strides(const std::vector<int>& shape) {
    std::vector<int> st(shape.size());
    int64_t v = 1;
    for (int i = (int)shape.size() - 1; i >= 0; --i) {
        st[i] = (int)v;
        v *= shape[i];
    }
    return st;
}

// ------------------------------------------------------------------ memory
namespace memory {

SynchronizedMemory::SynchronizedMemory(size_t bytes, bool pinned_host) : bytes_(bytes), pinned_host_(pinned_host) {}

SynchronizedMemory::~SynchronizedMemory() {
    // transfers in flight still use both blocks
    for (void* ev : {to_device_event_, to_host_event_})
        if (ev) {
            dali_hip_event_synchronize(ev);
            dali_hip_event_destroy(ev);
        }
    if (host_) {
        if (pinned_host_) dali_hip_host_free(host_);
        else std::free(host_);
    }
    // device blocks go back to the size-keyed bank, not to the driver
    // (dali/array/memory/synchronized_memory.cpp:76-82)
    if (device_) dali_hip_bank_deposit(device_, bytes_);
}

// Before a side is handed out: a transfer towards the device makes the compute stream wait for it (once); a
// transfer towards the host, or away from a host block that is about to be written, makes the host wait.
void SynchronizedMemory::settle(DeviceT device, bool host_will_write) {
    auto retire = [](void*& ev) {
        check_hip(dali_hip_event_destroy(ev), "event destroy");
        ev = nullptr;
    };
    if (device == DEVICE_T_GPU) {
        // a transfer that has not finished yet is put in front of whatever the compute stream does next with the
        // device block (a copy to the host still reads it, a copy from the host still writes it)
        for (void** ev : {&to_device_event_, &to_host_event_}) {
            if (!*ev) continue;
            int done = 0;
            check_hip(dali_hip_event_query(*ev, &done), "event query");
            if (done) {
                if (ev == &to_device_event_) retire(*ev);  // the host block is free again as well
                else continue;                             // the host side retires its own event when it reads
            } else {
                check_hip(dali_hip_stream_wait_event(*ev), "wait for migration");
            }
        }
    } else {
        if (to_host_event_) {
            check_hip(dali_hip_event_synchronize(to_host_event_), "wait for migration");
            retire(to_host_event_);
        }
        if (to_device_event_ && host_will_write) {
            check_hip(dali_hip_event_synchronize(to_device_event_), "wait for migration");
            retire(to_device_event_);
        }
    }
}

void SynchronizedMemory::prefetch(DeviceT device) {
    bool& fresh = device == DEVICE_T_CPU ? host_fresh_ : device_fresh_;
    if (fresh) return;
    const bool other_fresh = device == DEVICE_T_CPU ? device_fresh_ : host_fresh_;
    if (!pinned_host_ || !other_fresh) {
        move_to(device);
        return;
    }
    allocate(device);
    void*& slot = device == DEVICE_T_CPU ? to_host_event_ : to_device_event_;
    if (slot) {
        check_hip(dali_hip_event_synchronize(slot), "wait for migration");
        check_hip(dali_hip_event_destroy(slot), "event destroy");
        slot = nullptr;
    }
    void* ev = nullptr;
    check_hip(dali_hip_event_create(&ev), "event create");
    if (device == DEVICE_T_GPU) check_hip(dali_hip_memcpy_h2d_async(device_, host_, bytes_, ev), "asynchronous copy to device");
    else check_hip(dali_hip_memcpy_d2h_async(host_, device_, bytes_, ev), "asynchronous copy to host");
    slot = ev;
    fresh = true;
}

void SynchronizedMemory::lazy_clear() {
    clear_on_allocation_ = true;
    host_fresh_ = false;
    device_fresh_ = false;
    if (host_) {
        std::memset(host_, 0, bytes_);
        host_fresh_ = true;
    }
    if (device_) {
        check_hip(dali_hip_memset_async(device_, 0, bytes_), "memory clear");
        device_fresh_ = true;
    }
}

void SynchronizedMemory::allocate(DeviceT device) {
    if (device == DEVICE_T_CPU) {
        if (host_) return;
        size_t n = bytes_ ? bytes_ : 4;
        if (pinned_host_) check_hip(dali_hip_host_alloc(&host_, n), "pinned host allocation");
        else if (posix_memalign(&host_, 64, n) != 0) throw std::runtime_error("host allocation failed");
    } else {
        if (device_) return;
        check_hip(dali_hip_bank_allocate(&device_, bytes_), "device allocation");
    }
}

void SynchronizedMemory::move_to(DeviceT device) {
    bool& fresh = device == DEVICE_T_CPU ? host_fresh_ : device_fresh_;
    if (fresh) return;
    allocate(device);
    bool other_fresh = device == DEVICE_T_CPU ? device_fresh_ : host_fresh_;
    if (other_fresh) {
        if (device == DEVICE_T_CPU)
            check_hip(dali_hip_memcpy_d2h(host_, device_, bytes_), "copy to host");
        else
            check_hip(dali_hip_memcpy_h2d(device_, host_, bytes_), "copy to device");
    } else if (clear_on_allocation_) {
        if (device == DEVICE_T_CPU)
            std::memset(host_, 0, bytes_);
        else
            check_hip(dali_hip_memset_async(device_, 0, bytes_), "memory clear");
    }
    fresh = true;
}

const void* SynchronizedMemory::readonly_data(DeviceT device) {
    move_to(device);
    settle(device, false);
    return device == DEVICE_T_CPU ? host_ : device_;
}

void* SynchronizedMemory::mutable_data(DeviceT device) {
    move_to(device);
    settle(device, true);
    host_fresh_ = device == DEVICE_T_CPU;
    device_fresh_ = device == DEVICE_T_GPU;
    return device == DEVICE_T_CPU ? host_ : device_;
}

void* SynchronizedMemory::overwrite_data(DeviceT device) {
    allocate(device);
    settle(device, true);
    host_fresh_ = device == DEVICE_T_CPU;
    device_fresh_ = device == DEVICE_T_GPU;
    return device == DEVICE_T_CPU ? host_ : device_;
}

void* SynchronizedMemory::data(DeviceT device, AM mode) {
    switch (mode) {
        case AM_READONLY: return const_cast<void*>(readonly_data(device));
        case AM_MUTABLE: return mutable_data(device);
        default: return overwrite_data(device);
    }
}
}  // namespace memory

// ------------------------------------------------------------------- Array
static std::shared_ptr<Expr> make_buffer(const std::vector<int>& shape, DType dtype) {
    for (int s : shape) DALI_ASSERT(s >= 0, make_message("negative dimension in shape ", shape_str(shape)));
    auto e = std::make_shared<Expr>();
    e->kind = Kind::BUFFER;
    e->dtype = dtype;
    e->shape = shape;
    int64_t n = 1;
    for (int s : shape) n *= s;
    DALI_ASSERT(n < ((int64_t)1 << 31), make_message("array of shape ", shape_str(shape), " has too many elements"));
    e->memory = std::make_shared<memory::SynchronizedMemory>((size_t)n * size_of_dtype(dtype));
    return e;
}

Array::Array() : state_(nullptr) {}
Array::Array(std::shared_ptr<Expr> expr) : state_(std::make_shared<ArrayState>()) { state_->expr = std::move(expr); }
Array::Array(const std::vector<int>& shape, DType dtype) : Array(make_buffer(shape, dtype)) {}

static std::shared_ptr<Expr> make_scalar(DType dtype, double d, int i) {
    auto e = std::make_shared<Expr>();
    e->kind = Kind::SCALAR;
    e->dtype = dtype;
    e->dvalue = d;
    e->ivalue = i;
    return e;
}
Array::Array(double scalar) : Array(make_scalar(DTYPE_DOUBLE, scalar, (int)scalar)) {}
Array::Array(float scalar) : Array(make_scalar(DTYPE_FLOAT, scalar, (int)scalar)) {}
Array::Array(int scalar) : Array(make_scalar(DTYPE_INT32, scalar, scalar)) {}

Array Array::zeros(const std::vector<int>& shape, DType dtype) {
    Array a(shape, dtype);
    a.state_->expr->memory->lazy_clear();
    return a;
}

Array Array::from_host(const void* data, const std::vector<int>& shape, DType dtype) {
    Array a(shape, dtype);
    auto& mem = a.state_->expr->memory;
    void* dst = mem->overwrite_data(memory::DEVICE_T_CPU);
    std::memcpy(dst, data, mem->bytes());
    return a;
}

Array Array::from_host_pinned(const void* data, const std::vector<int>& shape, DType dtype) {
    Array a(shape, dtype);
    auto& e = a.state_->expr;
    e->memory = std::make_shared<memory::SynchronizedMemory>((size_t)e->numel() * size_of_dtype(dtype), true);
    std::memcpy(e->memory->overwrite_data(memory::DEVICE_T_CPU), data, e->memory->bytes());
    return a;
}

template <typename T>
static Array filled(const std::vector<int>& shape, DType dtype, bool ramp) {
    Array a(shape, dtype);
    auto& mem = a.state_->expr->memory;
    T* dst = (T*)mem->overwrite_data(memory::DEVICE_T_CPU);
    size_t n = mem->bytes() / sizeof(T);
    for (size_t i = 0; i < n; ++i) dst[i] = ramp ? (T)i : (T)1;
    return a;
}

Array Array::ones(const std::vector<int>& shape, DType dtype) {
    if (dtype == DTYPE_FLOAT) return filled<float>(shape, dtype, false);
    if (dtype == DTYPE_DOUBLE) return filled<double>(shape, dtype, false);
    return filled<int>(shape, dtype, false);
}

Array Array::arange(int n, DType dtype) {
    if (dtype == DTYPE_FLOAT) return filled<float>({n}, dtype, true);
    if (dtype == DTYPE_DOUBLE) return filled<double>({n}, dtype, true);
    return filled<int>({n}, dtype, true);
}

bool Array::is_stateless() const { return !state_ || !state_->expr; }
std::shared_ptr<Expr> Array::expression() const {
    DALI_ASSERT(!is_stateless(), "operation on a stateless Array");
    return state_->expr;
}
bool Array::is_buffer() const { return expression()->kind == Kind::BUFFER; }
bool Array::is_scalar() const { return expression()->shape.empty(); }
const std::vector<int>& Array::shape() const { return expression()->shape; }
int Array::ndim() const { return (int)expression()->shape.size(); }
DType Array::dtype() const { return expression()->dtype; }
int Array::number_of_elements() const { return expression()->numel(); }
const std::vector<int>& Array::strides() const { return expression()->strides; }
std::vector<int> Array::normalized_strides() const {
    auto e = expression();
    return e->strides.empty() ? contiguous_strides(e->shape) : e->strides;
}
int Array::offset() const { return expression()->offset; }

bool Array::contiguous_memory() const {
    auto e = expression();
    if (e->kind != Kind::BUFFER) return true;
    if (e->strides.empty()) return true;
    auto c = contiguous_strides(e->shape);
    for (size_t i = 0; i < c.size(); ++i)
        if (e->shape[i] != 1 && e->strides[i] != c[i]) return false;
    return true;
}

void Array::eval() const {
    if (is_buffer() || expression()->kind == Kind::SCALAR) return;
    evaluate({*this});
}

void Array::eval_together(const std::vector<Array>& roots) { evaluate(roots); }

static Array buffer_view(const std::shared_ptr<Expr>& base, const std::vector<int>& shape,
                         const std::vector<int>& strides, int offset) {
    auto e = std::make_shared<Expr>();
    e->kind = Kind::BUFFER;
    e->dtype = base->dtype;
    e->memory = base->memory;
    e->shape = shape;
    e->offset = offset;
    // store no strides when the view is contiguous (the reference's convention,
    // dali/array/expression/buffer.cpp:112-175)
    auto c = contiguous_strides(shape);
    bool contiguous = true;
    for (size_t i = 0; i < shape.size(); ++i)
        if (shape[i] != 1 && strides[i] != c[i]) contiguous = false;
    if (!contiguous) e->strides = strides;
    return Array(e);
}

// a scalar literal viewed as a buffer is materialised first
static const Array& as_buffer(const Array& a) {
    if (a.expression()->kind == Kind::SCALAR) {
        auto e = a.expression();
        Array b({}, e->dtype);
        void* p = b.expression()->memory->overwrite_data(memory::DEVICE_T_CPU);
        if (e->dtype == DTYPE_FLOAT) *(float*)p = (float)e->dvalue;
        else if (e->dtype == DTYPE_DOUBLE) *(double*)p = e->dvalue;
        else *(int*)p = e->ivalue;
        a.state_->expr = b.expression();
        return a;
    }
    a.eval();
    return a;
}

void Array::prefetch_to_device() const { as_buffer(*this).expression()->memory->prefetch(memory::DEVICE_T_GPU); }
void Array::prefetch_to_host() const { as_buffer(*this).expression()->memory->prefetch(memory::DEVICE_T_CPU); }

Array Array::transpose() const {
    std::vector<int> axes(ndim());
    for (int i = 0; i < ndim(); ++i) axes[i] = ndim() - 1 - i;
    return transpose(axes);
}

Array Array::transpose(const std::vector<int>& axes) const {
    DALI_ASSERT((int)axes.size() == ndim(), make_message("transpose needs ", ndim(), " axes (got ", axes.size(), ")."));
    if (expression()->kind == Kind::EXPAND_DIMS) {
        // Inserted unit axes over a lazy node (a keepdims reduction): when the permutation only moves the inserted axes
        // among the others, the result is the same node with the unit axes inserted elsewhere, still lazy.
        const int nd = ndim();
        std::vector<int> frame(nd);
        std::iota(frame.begin(), frame.end(), 0);
        std::vector<bool> inserted(nd, false);
        Array base = *this;
        while (base.expression()->kind == Kind::EXPAND_DIMS) {
            const int k = base.expression()->axis;
            inserted[frame[k]] = true;
            frame.erase(frame.begin() + k);
            base = base.expression()->args[0];
        }
        std::vector<int> kept_order;
        bool valid = true;
        std::vector<int> norm(nd);
        for (int i = 0; i < nd; ++i) {
            norm[i] = axes[i] < 0 ? axes[i] + nd : axes[i];
            valid = valid && norm[i] >= 0 && norm[i] < nd;
            if (valid && !inserted[norm[i]]) kept_order.push_back(norm[i]);
        }
        if (valid && kept_order == frame) {
            Array out = base;
            for (int i = 0; i < nd; ++i)
                if (inserted[norm[i]]) out = out.expand_dims(i);
            return out;
        }
    }
    {
        // An elementwise node over operands of its own shape (and literals) stays lazy: its transpose is the same node
        // over the transposed operands, so a reduction along a leading axis of an expression still fuses with it.
        auto le = expression();
        if (le->kind == Kind::ELEMENTWISE && ndim() >= 2) {
            bool movable = true;
            // (an operand broadcast from [.., 1, ..] moves as the broadcast of its transposed source)
            auto broadcast_of_same_rank = [&](const Array& x) {
                return x.expression()->kind == Kind::BROADCAST && x.expression()->args[0].ndim() == ndim();
            };
            for (const Array& x : le->args)
                movable = movable && (x.shape() == le->shape || x.expression()->kind == Kind::SCALAR) &&
                          (x.is_buffer() || x.expression()->kind == Kind::SCALAR || x.expression()->kind == Kind::ELEMENTWISE ||
                           x.expression()->kind == Kind::EXPAND_DIMS || broadcast_of_same_rank(x));
            if (movable) {
                std::vector<int> tshape(ndim());
                for (int i = 0; i < ndim(); ++i) tshape[i] = le->shape[axes[i] < 0 ? axes[i] + ndim() : axes[i]];
                std::vector<Array> targs;
                for (const Array& x : le->args) {
                    if (x.expression()->kind == Kind::SCALAR) targs.push_back(x);
                    else if (broadcast_of_same_rank(x)) {
                        auto bn = std::make_shared<Expr>(*x.expression());
                        bn->args = {x.expression()->args[0].transpose(axes)};
                        bn->shape = tshape;
                        targs.push_back(Array(bn));
                    }
                    else targs.push_back(x.transpose(axes));
                }
                auto n = std::make_shared<Expr>(*le);
                n->args = targs;
                for (const Array& t : targs)
                    if (t.expression()->kind != Kind::SCALAR) n->shape = t.shape();
                return Array(n);
            }
        }
    }
    auto e = as_buffer(*this).expression();
    auto st = normalized_strides();
    std::vector<int> nshape(ndim()), nstrides(ndim());
    std::vector<bool> seen(ndim(), false);
    for (int i = 0; i < ndim(); ++i) {
        int ax = axes[i] < 0 ? axes[i] + ndim() : axes[i];
        DALI_ASSERT(ax >= 0 && ax < ndim() && !seen[ax], "transpose axes must be a permutation");
        seen[ax] = true;
        nshape[i] = e->shape[ax];
        nstrides[i] = st[ax];
    }
    return buffer_view(e, nshape, nstrides, e->offset);
}

Array Array::swapaxes(int a, int b) const {
    std::vector<int> axes(ndim());
    std::iota(axes.begin(), axes.end(), 0);
    if (a < 0) a += ndim();
    if (b < 0) b += ndim();
    DALI_ASSERT(a >= 0 && a < ndim() && b >= 0 && b < ndim(), "swapaxes axis out of range");
    std::swap(axes[a], axes[b]);
    return transpose(axes);
}

Array Array::pluck_axis(int axis, int idx) const {
    if (axis < 0) axis += ndim();
    DALI_ASSERT(axis >= 0 && axis < ndim(), make_message("pluck_axis axis ", axis, " out of range for ndim ", ndim()));
    auto e = as_buffer(*this).expression();
    if (idx < 0) idx += e->shape[axis];
    DALI_ASSERT(idx >= 0 && idx < e->shape[axis], make_message("index ", idx, " out of range for axis of size ", e->shape[axis]));
    auto st = normalized_strides();
    std::vector<int> nshape, nstrides;
    for (int i = 0; i < ndim(); ++i)
        if (i != axis) {
            nshape.push_back(e->shape[i]);
            nstrides.push_back(st[i]);
        }
    return buffer_view(e, nshape, nstrides, e->offset + idx * st[axis]);
}

Array Array::slice(int axis, int start, int end, int step) const {
    if (axis < 0) axis += ndim();
    DALI_ASSERT(axis >= 0 && axis < ndim(), make_message("slice axis ", axis, " out of range for ndim ", ndim()));
    DALI_ASSERT(step != 0, "slice step cannot be zero");
    auto e = as_buffer(*this).expression();
    int n = e->shape[axis];
    if (start < 0) start += n;
    if (end < 0) end += n;
    DALI_ASSERT(start >= 0 && start <= n && end >= start && end <= n,
                make_message("slice [", start, ":", end, "] out of range for axis of size ", n));
    auto st = normalized_strides();
    std::vector<int> nshape = e->shape, nstrides = st;
    // dali/array/slice.cpp:76-81, dali/array/expression/buffer.cpp:177-209: ceil((end - start) / |step|) elements; a negative
    // step walks the same range [start, end) from its last element down, i.e. the view starts at end - 1
    const int astep = step < 0 ? -step : step;
    nshape[axis] = (end - start + astep - 1) / astep;
    nstrides[axis] = st[axis] * step;
    const int first = step > 0 || end == start ? start : end - 1;
    return buffer_view(e, nshape, nstrides, e->offset + first * st[axis]);
}

Array Array::ascontiguousarray() const {
    const Array& self = as_buffer(*this);
    if (self.contiguous_memory()) return self;
    Array out(shape(), dtype());
    evaluate_into(out, OPERATOR_T_EQL, op::identity(self));
    return out;
}

Array Array::reshape(const std::vector<int>& new_shape) const {
    std::vector<int> ns = new_shape;
    int64_t known = 1;
    int unknown = -1;
    for (size_t i = 0; i < ns.size(); ++i) {
        if (ns[i] == -1) {
            DALI_ASSERT(unknown < 0, "reshape accepts at most one -1");
            unknown = (int)i;
        } else {
            known *= ns[i];
        }
    }
    if (unknown >= 0) ns[unknown] = known ? (int)(number_of_elements() / known) : 0;
    int64_t total = 1;
    for (int s : ns) total *= s;
    DALI_ASSERT(total == number_of_elements(), make_message("cannot reshape ", shape_str(shape()), " into ", shape_str(new_shape)));
    Array src = as_buffer(*this).contiguous_memory() ? *this : ascontiguousarray();
    auto e = src.expression();
    return buffer_view(e, ns, contiguous_strides(ns), e->offset);
}

Array Array::expand_dims(int axis) const {
    if (axis < 0) axis += ndim() + 1;
    DALI_ASSERT(axis >= 0 && axis <= ndim(), make_message("expand_dims axis ", axis, " out of range for ndim ", ndim()));
    auto e = expression();
    if (e->kind == Kind::BUFFER) {
        auto st = normalized_strides();
        std::vector<int> nshape = e->shape, nstrides = st;
        nshape.insert(nshape.begin() + axis, 1);
        nstrides.insert(nstrides.begin() + axis, 0);
        return buffer_view(e, nshape, nstrides, e->offset);
    }
    auto n = std::make_shared<Expr>();
    n->kind = Kind::EXPAND_DIMS;
    n->dtype = e->dtype;
    n->shape = e->shape;
    n->shape.insert(n->shape.begin() + axis, 1);
    n->axis = axis;
    n->args = {*this};
    return Array(n);
}

Array Array::squeeze(int axis) const {
    if (axis < 0) axis += ndim();
    DALI_ASSERT(axis >= 0 && axis < ndim() && shape()[axis] == 1,
                make_message("squeeze axis ", axis, " must have size 1 in shape ", shape_str(shape())));
    return pluck_axis(axis, 0);
}

void* Array::device_ptr(memory::AM mode) const {
    auto e = as_buffer(*this).expression();
    char* base = (char*)e->memory->data(memory::DEVICE_T_GPU, mode);
    return base + (size_t)e->offset * size_of_dtype(e->dtype);
}

void Array::to_host(void* out) const {
    auto e = as_buffer(*this).expression();
    const char* src = (const char*)e->memory->readonly_data(memory::DEVICE_T_CPU);
    int es = size_of_dtype(e->dtype);
    int n = e->numel();
    if (n == 0) return;
    if (contiguous_memory()) {
        std::memcpy(out, src + (size_t)e->offset * es, (size_t)n * es);
        return;
    }
    auto st = normalized_strides();
    int nd = ndim();
    std::vector<int> idx(nd, 0);
    char* dst = (char*)out;
    for (int i = 0; i < n; ++i) {
        int64_t off = e->offset;
        for (int d = 0; d < nd; ++d) off += (int64_t)idx[d] * st[d];
        std::memcpy(dst + (size_t)i * es, src + off * es, es);
        for (int d = nd - 1; d >= 0; --d) {
            if (++idx[d] < e->shape[d]) break;
            idx[d] = 0;
        }
    }
}

double Array::scalar_value() const {
    auto e = expression();
    if (e->kind == Kind::SCALAR) return e->dtype == DTYPE_INT32 ? (double)e->ivalue : e->dvalue;
    DALI_ASSERT(number_of_elements() >= 1, "scalar_value of an empty array");
    auto b = as_buffer(*this).expression();
    const char* src = (const char*)b->memory->readonly_data(memory::DEVICE_T_CPU) + (size_t)b->offset * size_of_dtype(b->dtype);
    if (b->dtype == DTYPE_FLOAT) return *(const float*)src;
    if (b->dtype == DTYPE_DOUBLE) return *(const double*)src;
    return *(const int*)src;
}

Array& Array::assign(const Array& other) {
    if (is_stateless()) {
        other.eval();
        state_ = std::make_shared<ArrayState>();
        state_->expr = other.expression();
        return *this;
    }
    evaluate_into(*this, OPERATOR_T_EQL, other);
    return *this;
}
Array& Array::operator+=(const Array& other) { evaluate_into(*this, OPERATOR_T_ADD, other); return *this; }
Array& Array::operator-=(const Array& other) { evaluate_into(*this, OPERATOR_T_SUB, other); return *this; }
Array& Array::operator*=(const Array& other) { evaluate_into(*this, OPERATOR_T_MUL, other); return *this; }
Array& Array::operator/=(const Array& other) { evaluate_into(*this, OPERATOR_T_DIV, other); return *this; }
Array& Array::operator<<=(const Array& other) { return op::autoreduce_assign(*this, other); }
Array Array::operator[](const Array& indices) const { return op::gather(*this, indices); }
Array Array::gather_from_rows(const Array& indices) const { return op::gather_from_rows(*this, indices); }

Array Array::sum() const { return op::sum(*this); }
Array Array::sum(const std::vector<int>& axes, bool keepdims) const { return op::sum(*this, axes, keepdims); }
Array Array::max() const { return op::max(*this); }
Array Array::max(const std::vector<int>& axes, bool keepdims) const { return op::max(*this, axes, keepdims); }
Array Array::min() const { return op::min(*this); }
Array Array::min(const std::vector<int>& axes, bool keepdims) const { return op::min(*this, axes, keepdims); }
Array Array::mean() const { return op::mean(*this); }
Array Array::mean(const std::vector<int>& axes, bool keepdims) const { return op::mean(*this, axes, keepdims); }
Array Array::argmax() const { return op::argmax(*this); }
Array Array::argmax(int axis) const { return op::argmax(*this, axis); }
Array Array::argmin() const { return op::argmin(*this); }
Array Array::argmin(int axis) const { return op::argmin(*this, axis); }
Array Array::exp() const { return op::exp(*this); }
Array Array::log() const { return op::log(*this); }
Array Array::tanh() const { return op::tanh(*this); }
Array Array::sigmoid() const { return op::sigmoid(*this); }
Array Array::square() const { return op::square(*this); }
Array Array::dot(const Array& other) const { return op::dot(*this, other); }

Array operator+(const Array& a, const Array& b) { return op::add(a, b); }
Array operator-(const Array& a, const Array& b) { return op::subtract(a, b); }
Array operator*(const Array& a, const Array& b) { return op::eltmul(a, b); }
Array operator/(const Array& a, const Array& b) { return op::eltdiv(a, b); }
Array operator-(const Array& a) { return op::negate(a); }

// --------------------------------------------------------------------- op::
namespace op {

static Array make_node(Kind kind, const std::string& name, std::vector<Array> args, const std::vector<int>& shape,
                       DType dtype) {
    auto e = std::make_shared<Expr>();
    e->kind = kind;
    e->name = name;
    e->args = std::move(args);
    e->shape = shape;
    e->dtype = dtype;
    return Array(e);
}

// dali/array/array.cpp:845-865
static DType type_promotion(const Array& a, const Array& b) {
    bool as = a.is_scalar(), bs = b.is_scalar();
    if (as == bs) {
        if (a.dtype() == DTYPE_DOUBLE || b.dtype() == DTYPE_DOUBLE) return DTYPE_DOUBLE;
        if (a.dtype() == DTYPE_FLOAT || b.dtype() == DTYPE_FLOAT) return DTYPE_FLOAT;
        return DTYPE_INT32;
    }
    return as ? b.dtype() : a.dtype();
}

// dali/array/jit/jit_utils.cpp:107-147
static std::vector<int> common_shape(const Array& a, const Array& b) {
    const auto& sa = a.shape();
    const auto& sb = b.shape();
    if (sa.empty()) return sb;
    if (sb.empty()) return sa;
    DALI_ASSERT(sa.size() == sb.size(), "inputs must be scalars or have the same dimensionality.");
    std::vector<int> out = sa;
    for (size_t d = 0; d < sa.size(); ++d) {
        DALI_ASSERT(sa[d] == sb[d] || sa[d] == 1 || sb[d] == 1,
                    make_message("Could not find a common shape between ", shape_str(sa), " and ", shape_str(sb), "."));
        if (sb[d] != 1) out[d] = sb[d];
    }
    return out;
}

static Array broadcasted_reshape(const Array& a, const std::vector<int>& shape) {
    if (a.shape() == shape) return a;
    return make_node(Kind::BROADCAST, "", {a}, shape, a.dtype());
}

Array unsafe_cast(Array a, DType dtype) {
    if (a.dtype() == dtype) return a;
    auto e = a.expression();
    if (e->kind == Kind::SCALAR) {
        // literal: convert on the host
        if (dtype == DTYPE_INT32) return Array((int)(e->dtype == DTYPE_INT32 ? e->ivalue : e->dvalue));
        double v = e->dtype == DTYPE_INT32 ? (double)e->ivalue : e->dvalue;
        if (dtype == DTYPE_FLOAT) return Array((float)v);
        return Array(v);
    }
    return make_node(Kind::ELEMENTWISE, "functor::cast", {a}, a.shape(), dtype);
}

Array round(Array a) {
    if (a.dtype() == DTYPE_INT32) return a;
    auto e = a.expression();
    if (e->kind == Kind::SCALAR) return Array((int)std::floor(e->dvalue + 0.5));
    return make_node(Kind::ELEMENTWISE, "functor::round", {a}, a.shape(), DTYPE_INT32);
}

// dali/array/op/elementwise_operation.cpp:155-160 (the reference names a functor "ceiling" that functor.h:150-155 defines
// as "ceil"; the result is int32 like round's)
Array ceil(Array a) {
    if (a.dtype() == DTYPE_INT32) return a;
    auto e = a.expression();
    if (e->kind == Kind::SCALAR) return Array((int)std::ceil(e->dvalue));
    return make_node(Kind::ELEMENTWISE, "functor::ceil", {a}, a.shape(), DTYPE_INT32);
}

// dali/array/op/elementwise_operation.cpp:137-139
Array astype(Array a, DType dtype) { return dtype == DTYPE_INT32 ? round(a) : unsafe_cast(a, dtype); }

Array elementwise(Array a, const std::string& functor_name) {
    return make_node(Kind::ELEMENTWISE, functor_name, {a}, a.shape(), a.dtype());
}

// dali/array/op/elementwise_operation.cpp:130-135,162-186
Array elementwise(Array a, Array b, const std::string& functor_name) {
    DALI_ASSERT(a.ndim() == b.ndim() || a.is_scalar() || b.is_scalar(),
                make_message("Arguments to binary operation '", functor_name, "' must have the same rank (got left.ndim = ",
                             a.ndim(), ", left.shape = ", shape_str(a.shape()), ", and right.ndim = ", b.ndim(),
                             ", right.shape = ", shape_str(b.shape()), ")."));
    if (a.dtype() != b.dtype()) {
        DType t = type_promotion(a, b);
        a = astype(a, t);
        b = astype(b, t);
    }
    std::vector<int> shape = common_shape(a, b);
    if (!a.is_scalar()) a = broadcasted_reshape(a, shape);
    if (!b.is_scalar()) b = broadcasted_reshape(b, shape);
    return make_node(Kind::ELEMENTWISE, functor_name, {a, b}, shape, a.dtype());
}

Array add(const Array& a, const Array& b) { return elementwise(a, b, "functor::add"); }
Array subtract(const Array& a, const Array& b) { return elementwise(a, b, "functor::subtract"); }
Array eltmul(const Array& a, const Array& b) { return elementwise(a, b, "functor::eltmul"); }
Array eltdiv(const Array& a, const Array& b) { return elementwise(a, b, "functor::eltdiv"); }
Array pow(const Array& a, const Array& b) { return elementwise(a, b, "functor::power"); }
Array equals(const Array& a, const Array& b) { return elementwise(a, b, "functor::equals"); }
Array prelu(const Array& x, const Array& w) { return elementwise(x, w, "functor::prelu"); }
Array clip(const Array& x, const Array& c) { return elementwise(x, c, "functor::clip"); }
Array identity(const Array& x) { return elementwise(x, "functor::identity"); }
Array sigmoid(const Array& x) { return elementwise(x, "functor::sigmoid"); }
Array tanh(const Array& x) { return elementwise(x, "functor::tanh"); }
Array exp(const Array& x) { return elementwise(x, "functor::exp"); }
Array log(const Array& x) { return elementwise(x, "functor::log"); }
Array softplus(const Array& x) { return elementwise(x, "functor::softplus"); }
Array relu(const Array& x) { return elementwise(x, "functor::relu"); }
Array abs(const Array& x) { return elementwise(x, "functor::abs"); }
Array sign(const Array& x) { return elementwise(x, "functor::sign"); }
Array square(const Array& x) { return elementwise(x, "functor::square"); }
Array cube(const Array& x) { return elementwise(x, "functor::cube"); }
Array sqrt(const Array& x) { return elementwise(x, "functor::sqrt_f"); }
Array rsqrt(const Array& x) { return elementwise(x, "functor::rsqrt"); }
Array eltinv(const Array& x) { return elementwise(x, "functor::inv"); }
Array negate(const Array& x) { return eltmul(Array(-1), x); }
Array isnan(const Array& x) { return elementwise(x, "functor::isnotanumber"); }
Array isinf(const Array& x) { return elementwise(x, "functor::isinfinity"); }
Array dsigmoid(const Array& x) { return elementwise(x, "functor::dsigmoid"); }
Array dtanh(const Array& x) { return elementwise(x, "functor::dtanh"); }
// the rest of dali/array/op/unary.cpp and binary.cpp: thin names over the functors
Array softplus_backward(const Array& x) { return elementwise(x, "functor::softplus_backward"); }
Array relu_backward(const Array& x) { return elementwise(x, "functor::relu_backward"); }
Array log_or_zero(const Array& x) { return elementwise(x, "functor::log_or_zero"); }
Array inverse_tanh(const Array& x) { return elementwise(x, "functor::inverse_tanh"); }
Array clipped_relu(const Array& x, const Array& upper_bound) { return elementwise(x, upper_bound, "functor::clipped_relu"); }
Array clipped_relu_backward(const Array& x, const Array& upper_bound) { return elementwise(x, upper_bound, "functor::clipped_relu_backward"); }
Array steep_sigmoid(const Array& x, const Array& aggressiveness) { return elementwise(x, aggressiveness, "functor::steep_sigmoid"); }
Array steep_sigmoid_backward(const Array& x, const Array& aggressiveness) { return elementwise(x, aggressiveness, "functor::steep_sigmoid_backward"); }
Array prelu_backward_weights(const Array& a, const Array& grad) { return elementwise(a, grad, "functor::prelu_backward_weights"); }
Array prelu_backward_inputs(const Array& a, const Array& weights) { return elementwise(a, weights, "functor::prelu_backward_inputs"); }
Array lessthanequal(const Array& a, const Array& b) { return elementwise(a, b, "functor::lessthanequal"); }
Array greaterthanequal(const Array& a, const Array& b) { return elementwise(a, b, "functor::greaterthanequal"); }
Array maximum(const Array& a, const Array& b) { return elementwise(a, b, "functor::max_scalar"); }
Array minimum(const Array& a, const Array& b) { return elementwise(a, b, "functor::min_scalar"); }
Array binary_cross_entropy(const Array& a, const Array& b) { return elementwise(a, b, "functor::binary_cross_entropy"); }
Array binary_cross_entropy_grad(const Array& a, const Array& b) { return elementwise(a, b, "functor::binary_cross_entropy_grad"); }
Array close(const Array& left, const Array& right, const Array& atolerance) { return lessthanequal(abs(subtract(left, right)), atolerance); }
// dali/array/op/binary.cpp:9-11,45-60 (sum of many arrays as one fused chain)
Array add(const std::vector<Array>& arrays) {
    DALI_ASSERT(!arrays.empty(), "add must have at least one Array to add but got 0.");
    Array out = arrays[0];
    for (size_t i = 1; i < arrays.size(); ++i) out = add(out, arrays[i]);
    return out;
}

// A reduction over no elements is the reducer's initial value: the reference's loops never run and store what
// SetInitValue left (dali/array/jit/reducer_kernels.h:57-169, all_reduce_kernel_utils.cpp:105-154). No kernel is
// planned for it; the result is a buffer filled with that value.
static Array reduction_of_nothing(const std::vector<int>& shape, const std::string& reducer_name, DType dtype) {
    Array out(shape, dtype);
    if (out.number_of_elements() == 0) return out;
    if (reducer_name == "reducers::sum") return out.assign(Array(0));
    if (reducer_name == "reducers::product") return out.assign(Array(1));
    const bool is_max = reducer_name == "reducers::maximum";
    DALI_ASSERT(is_max || reducer_name == "reducers::minimum", make_message("reduction of an empty array by ", reducer_name));
    if (dtype == DTYPE_INT32) return out.assign(Array(is_max ? std::numeric_limits<int>::min() : std::numeric_limits<int>::max()));
    if (dtype == DTYPE_DOUBLE) return out.assign(Array(is_max ? -std::numeric_limits<double>::max() : std::numeric_limits<double>::max()));
    return out.assign(Array(is_max ? -std::numeric_limits<float>::max() : std::numeric_limits<float>::max()));
}

Array all_reduce(const Array& a, const std::string& reducer_name) {
    if (a.number_of_elements() == 0) return reduction_of_nothing({}, reducer_name, a.dtype());
    return make_node(Kind::ALL_REDUCE, reducer_name, {a}, {}, a.dtype());
}

static Array axis_reduce_last(const Array& a, const std::string& reducer_name) {
    std::vector<int> shape(a.shape().begin(), a.shape().end() - 1);
    if (a.shape().back() == 0) return reduction_of_nothing(shape, reducer_name, a.dtype());
    return make_node(Kind::AXIS_REDUCE, reducer_name, {a}, shape, a.dtype());
}

// true when buffer axis `axis` and `axis - 1` can be merged into one
// (dali/array/array.cpp is_axis_collapsible_with_axis_minus_one)
static bool collapsible_with_axis_minus_one(const Array& a, int axis) {
    if (!a.is_buffer()) return false;
    auto st = a.normalized_strides();
    return st[axis - 1] == st[axis] * a.shape()[axis];
}

static Array collapse_axis_with_axis_minus_one(const Array& a, int axis) {
    auto e = a.expression();
    auto st = a.normalized_strides();
    std::vector<int> nshape = e->shape, nstrides = st;
    nshape[axis - 1] *= nshape[axis];
    nstrides[axis - 1] = st[axis];
    nshape.erase(nshape.begin() + axis);
    nstrides.erase(nstrides.begin() + axis);
    return buffer_view(e, nshape, nstrides, e->offset);
}

// dali/array/op/reducer_operation.cpp:595-679
Array axis_reduce(const Array& a, const std::string& reducer_name, const std::vector<int>& axes, bool keepdims) {
    if (axes.empty()) return a;
    int ndim = a.ndim();
    if (ndim == 0) return a;
    std::vector<int> norm(axes);
    for (auto& ax : norm) {
        if (ax < 0) ax += ndim;
        DALI_ASSERT(ax >= 0 && ax < ndim,
                    make_message("Reduction axis must strictly positive and less than the number of dimensions of the input (got axis=",
                                 axes[0], ", ndim=", ndim, ", input.shape = ", shape_str(a.shape()), ")."));
    }
    std::vector<bool> reduced(ndim, false);
    std::sort(norm.begin(), norm.end());
    for (int ax : norm) {
        DALI_ASSERT(!reduced[ax], make_message("axis_reduce received duplicate axes to operate on (axis=", ax, ")."));
        reduced[ax] = true;
    }
    if ((int)norm.size() == ndim) return all_reduce(a, reducer_name);
    int num_low = 0;
    for (int i = ndim - 1; i >= 0 && reduced[i]; --i) ++num_low;
    if (num_low > 0 && num_low < (int)norm.size() && (reducer_name == "reducers::sum" || reducer_name == "reducers::maximum" ||
                                                      reducer_name == "reducers::minimum" || reducer_name == "reducers::product")) {
        // Some reduced axes trail, others do not (per-channel sums of [N, C, H*W]): the trailing ones are reduced where they
        // lie, along memory, and only the much smaller result takes the transposed route for the others. The reference
        // moves every reduced axis to the back first (reducer_operation.cpp:595-679), i.e. a strided walk over everything.
        std::vector<int> tail_axes, rest;
        for (int ax : norm) (ax >= ndim - num_low ? tail_axes : rest).push_back(ax);
        Array out = axis_reduce(axis_reduce(a, reducer_name, tail_axes, false), reducer_name, rest, false);
        if (keepdims)
            for (int ax : norm) out = out.expand_dims(ax);
        return out;
    }
    Array res = a;
    if (num_low != (int)norm.size()) {
        std::vector<int> order;
        for (int i = 0; i < ndim; ++i)
            if (!reduced[i]) order.push_back(i);
        for (int i = 0; i < ndim; ++i)
            if (reduced[i]) order.push_back(i);
        res = res.transpose(order);
    }
    int to_reduce = (int)norm.size();
    int collapsed_ndim = ndim - 1;
    for (int used = 0; used < to_reduce; ++used) {
        if (to_reduce - used == 1 || !collapsible_with_axis_minus_one(res, collapsed_ndim)) {
            res = axis_reduce_last(res, reducer_name);
        } else {
            res = collapse_axis_with_axis_minus_one(res, collapsed_ndim);
        }
        --collapsed_ndim;
    }
    if (keepdims)
        for (int ax : norm) res = res.expand_dims(ax);
    return res;
}

// The reference stores a flat argmax in the INPUT dtype
// (dali/array/op/reducer_operation.cpp:681-684).
Array argument_all_reduce(const Array& a, const std::string& reducer_name) {
    if (a.number_of_elements() == 0) return reduction_of_nothing({}, "reducers::sum", a.dtype());  // the index stays 0
    return make_node(Kind::ARG_ALL_REDUCE, reducer_name, {a}, {}, a.dtype());
}

// dali/array/op/reducer_operation.cpp:686-710
Array argument_axis_reduce(const Array& a, const std::string& reducer_name, int axis) {
    int ndim = a.ndim();
    if (ndim == 0) return Array(0);
    if (axis < 0) axis += ndim;
    DALI_ASSERT(axis >= 0 && axis < ndim,
                make_message("Reduction axis must strictly positive and less than the number of dimensions of the input (got axis=",
                             axis, ", ndim=", ndim, ")."));
    if (ndim == 1) return argument_all_reduce(a, reducer_name);
    Array res = a;
    if (axis != ndim - 1) res = res.swapaxes(axis, ndim - 1);
    std::vector<int> shape(res.shape().begin(), res.shape().end() - 1);
    if (res.shape().back() == 0) return reduction_of_nothing(shape, "reducers::sum", DTYPE_INT32);  // the index stays 0
    return make_node(Kind::ARG_AXIS_REDUCE, reducer_name, {res}, shape, DTYPE_INT32);
}

Array sum(const Array& x) { return all_reduce(x, "reducers::sum"); }
Array sum(const Array& x, const std::vector<int>& axes, bool keepdims) { return axis_reduce(x, "reducers::sum", axes, keepdims); }
Array prod(const Array& x) { return all_reduce(x, "reducers::product"); }
Array prod(const Array& x, const std::vector<int>& axes, bool keepdims) { return axis_reduce(x, "reducers::product", axes, keepdims); }
Array max(const Array& x) { return all_reduce(x, "reducers::maximum"); }
Array max(const Array& x, const std::vector<int>& axes, bool keepdims) { return axis_reduce(x, "reducers::maximum", axes, keepdims); }
Array min(const Array& x) { return all_reduce(x, "reducers::minimum"); }
Array min(const Array& x, const std::vector<int>& axes, bool keepdims) { return axis_reduce(x, "reducers::minimum", axes, keepdims); }

// dali/array/op/reducers.cpp:32-41
Array mean(const Array& x) {
    Array s = all_reduce(x, "reducers::sum");
    if (s.dtype() == DTYPE_INT32) s = astype(s, DTYPE_DOUBLE);
    return eltdiv(s, Array(x.number_of_elements()));
}
Array mean(const Array& x, const std::vector<int>& axes, bool keepdims) {
    Array s = axis_reduce(x, "reducers::sum", axes, keepdims);
    if (s.dtype() == DTYPE_INT32) s = astype(s, DTYPE_DOUBLE);
    int n = s.number_of_elements();
    return eltdiv(s, Array(n ? x.number_of_elements() / n : 0));
}
Array L2_norm(const Array& x) {
    Array s = all_reduce(square(x), "reducers::sum");
    if (s.dtype() == DTYPE_INT32) s = astype(s, DTYPE_DOUBLE);
    return sqrt(s);
}
Array L2_norm(const Array& x, const std::vector<int>& axes, bool keepdims) {
    Array s = axis_reduce(square(x), "reducers::sum", axes, keepdims);
    if (s.dtype() == DTYPE_INT32) s = astype(s, DTYPE_DOUBLE);
    return sqrt(s);
}
Array argmax(const Array& x) { return argument_all_reduce(x, "reducers::maximum"); }
Array argmax(const Array& x, int axis) { return argument_axis_reduce(x, "reducers::maximum", axis); }
Array argmin(const Array& x) { return argument_all_reduce(x, "reducers::minimum"); }
Array argmin(const Array& x, int axis) { return argument_axis_reduce(x, "reducers::minimum", axis); }
// dali/array/op/reducers.cpp:61-72, binary.cpp:7-12
Array any_isnan(const Array& x) { return max(isnan(x)); }
Array any_isinf(const Array& x) { return max(isinf(x)); }
Array any_isnan(const Array& x, const std::vector<int>& axes, bool keepdims) { return max(isnan(x), axes, keepdims); }
Array any_isinf(const Array& x, const std::vector<int>& axes, bool keepdims) { return max(isinf(x), axes, keepdims); }
Array all_equals(const Array& left, const Array& right) { return prod(equals(left, right)); }
Array all_close(const Array& left, const Array& right, const Array& atolerance) { return prod(close(left, right, atolerance)); }

// dali/array/op/softmax.cpp:5-8
Array softmax_naive(const Array& logits, int axis) {
    Array exped = exp(subtract(logits, max(logits, {axis}, true)));
    return eltdiv(exped, sum(exped, {axis}, true));
}
// The same expression, kept as one node until it is evaluated: the planner then writes it out as above, or, for shapes
// that starve the fused row kernel (few very long rows, an axis that runs against memory), computes the maxima and the
// sums of exponentials in a pass of their own first.
Array softmax(const Array& logits, int axis) {
    const int nd = logits.ndim();
    const int ax = axis < 0 ? axis + nd : axis;
    if (nd == 0 || ax < 0 || ax >= nd || logits.dtype() == DTYPE_INT32 || logits.number_of_elements() == 0)
        return softmax_naive(logits, axis);  // (raises the reduction's own error for a bad axis)
    Array out = make_node(Kind::SOFTMAX, "", {logits}, logits.shape(), logits.dtype());
    out.expression()->axis = ax;
    return out;
}

// dali/array/op/softmax.cpp:10-13: the reference does not read `temperature`; the result is softmax(logits, axis)
Array softmax_temperature(const Array& logits, const Array& temperature, int axis) {
    (void)temperature;
    return softmax(logits, axis);
}

// dali/array/op/gather_from_rows.cpp:110-127
Array gather_from_rows(const Array& source, const Array& indices) {
    DALI_ASSERT(source.ndim() > 1, make_message("gather must be called on source with ndim >= 2 (got ndim=", source.ndim(), ")."));
    DALI_ASSERT(indices.dtype() == DTYPE_INT32, "indices must be integers.");
    DALI_ASSERT(indices.ndim() <= 1, make_message("indices must have rank 1 or lower (got indices.ndim=", indices.ndim(), ")."));
    DALI_ASSERT(source.ndim() == 2, "gather_from_rows: only 2-D sources are implemented");
    if (indices.ndim() == 1) {
        DALI_ASSERT(indices.shape()[0] <= source.shape()[0] || indices.shape()[0] == 1 || source.shape()[0] == 1,
                    make_message("dimension 1 of indices must be less than or equal to first dimension of source (got indices.shape[0]=",
                                 indices.shape()[0], ", source.shape[0]=", source.shape()[0], ")"));
    }
    std::vector<int> shape = indices.ndim() ? indices.shape() : std::vector<int>{1};
    return make_node(Kind::GATHER_FROM_ROWS, "", {source, indices}, shape, source.dtype());
}

// dali/array/op/gather.cpp:163-171: out[i..., rest...] = source[indices[i...], rest...]. The node keeps the
// source as a 2-D [V, D] view and the indices as a 1-D vector; its own shape is indices.shape + source.shape[1:].
// Assigning to the lazy node scatters into the source buffer (gather.cpp:126-143).
Array gather(const Array& source, const Array& indices) {
    DALI_ASSERT(source.ndim() > 0, make_message("gather must be called on source with ndim > 0 (got ndim=", source.ndim(), ")."));
    DALI_ASSERT(indices.dtype() == DTYPE_INT32, make_message("indices must be integers (got dtype=", dtype_to_cpp_name(indices.dtype()), ")."));
    Array src2 = source;
    if (source.ndim() == 1) src2 = source.expand_dims(1);
    else if (source.ndim() > 2) src2 = source.reshape({source.shape()[0], -1});
    Array idx1 = indices.ndim() == 1 ? indices : indices.reshape({-1});
    std::vector<int> shape = indices.shape();
    shape.insert(shape.end(), source.shape().begin() + 1, source.shape().end());
    Array node = make_node(Kind::GATHER, "", {src2, idx1}, shape, source.dtype());
    if (source.ndim() > 2 && source.is_buffer() && !(src2.is_buffer() && src2.expression()->memory == source.expression()->memory))
        node.expression()->origin = {source};  // the [V, D] form is a copy: assignments go through the view (jit_scatter.cpp)
    return node;
}

// dali/array/expression/assignment.cpp:92-126: left += sum of right over the axes where left has extent 1
Array& autoreduce_assign(Array& left, const Array& right) {
    DALI_ASSERT(left.ndim() == right.ndim(), make_message("destination for autoreduce_assign must have the same dimensionality as the input (destination.ndim = ",
                                                          left.ndim(), " vs input.ndim = ", right.ndim()));
    std::vector<int> reduction_axes;
    for (int i = 0; i < right.ndim(); ++i) {
        if (left.shape()[i] != right.shape()[i]) {
            DALI_ASSERT(left.shape()[i] == 1, make_message("Could not autoreduce_assign: destination must have all dimensions equal input dimensions or equal 1, but destination.shape[",
                                                           i, "] = ", left.shape()[i], " vs input.shape[", i, "] = ", right.shape()[i]));
            reduction_axes.push_back(i);
        }
    }
    Array r = reduction_axes.empty() ? right : sum(right, reduction_axes, /*keepdims=*/true);
    left += r;
    return left;
}

// dali/array/op/scan.cpp:183-194
Array axis_scan(const Array& a, const std::string& reducer_name, bool inclusive) {
    std::vector<int> shape = a.shape();
    if (!inclusive) {
        if (shape.empty()) shape = {2};
        else shape.back() += 1;
    }
    Array n = make_node(Kind::AXIS_SCAN, reducer_name, {a}, shape, a.dtype());
    n.expression()->depth = inclusive ? 1 : 0;
    return n;
}
Array cumsum(const Array& a, bool inclusive) { return axis_scan(a, "reducers::sum", inclusive); }
Array cumprod(const Array& a, bool inclusive) { return axis_scan(a, "reducers::product", inclusive); }

// dali/array/op/arange.cpp:41-57
Array arange(const Array& start, const Array& stop, const Array& step) {
    DALI_ASSERT(start.ndim() == 0, make_message("arange's start argument must be a scalar but got start.shape = ", shape_str(start.shape()), "."));
    DALI_ASSERT(stop.ndim() == 0, make_message("arange's stop argument must be a scalar but got stop.shape = ", shape_str(stop.shape()), "."));
    DALI_ASSERT(step.ndim() == 0, make_message("arange's step argument must be a scalar but got step.shape = ", shape_str(step.shape()), "."));
    const double b = start.scalar_value(), e = stop.scalar_value(), st = step.scalar_value();
    const int size = (int)std::ceil((e - b) / st);
    DALI_ASSERT(size > 0, make_message("arange's size must be strictly positive (got start = ", b, ", stop = ", e, ", step = ", st, ")."));
    return make_node(Kind::ARANGE, "", {start, step}, {size}, start.dtype());
}
Array arange(int start, int stop) { return arange(Array(start), Array(stop), Array(1)); }
Array arange(int size) { return arange(0, size); }

// dali/array/op/eye.cpp:46-77
Array diag(const Array& array, int rows, int cols) {
    DALI_ASSERT(rows > 0 && cols > 0, make_message("diag's rows and cols must > 0 (got rows = ", rows, ", cols = ", cols, ")."));
    DALI_ASSERT(array.ndim() <= 1, make_message("diag's argument must be a scalar or a vector (got array.shape = ", shape_str(array.shape()), ")."));
    if (array.ndim() == 1) {
        DALI_ASSERT(array.shape()[0] >= std::min(rows, cols), make_message("diag's argument is smaller than the maximal diagonal item (array.shape = ",
                                                                           shape_str(array.shape()), ", rows = ", rows, ", cols = ", cols, ")."));
    }
    return make_node(Kind::DIAG, "", {array}, {rows, cols}, array.dtype());
}
Array diag(const Array& array, int rows) { return diag(array, rows, rows); }
Array diag(const Array& array) {
    DALI_ASSERT(array.ndim() == 1, "diag without an extent needs a vector");
    return diag(array, array.shape()[0], array.shape()[0]);
}
Array eye(int rows, int cols) {
    DALI_ASSERT(rows > 0 && cols > 0, make_message("eye's rows and cols must > 0 (got rows = ", rows, ", cols = ", cols, ")."));
    return diag(Array(1.0f), rows, cols);
}
Array eye(int size) { return eye(size, size); }

// dali/array/op/outer.cpp:8-36: out[i, j] = a[i] * b[j], expressed through the broadcasting elementwise map
Array outer(const Array& a, const Array& b) {
    DALI_ASSERT(a.ndim() == 1 && b.ndim() == 1, make_message("outer takes two vectors (got a.ndim = ", a.ndim(), ", b.ndim = ", b.ndim(), ")."));
    return eltmul(a.expand_dims(1), b.expand_dims(0));
}

// dali/array/op/circular_convolution.cpp:82-86: out[..., x] = sum_s content[..., (x + s) mod n] * weights[..., s]
Array circular_convolution(Array x, Array weights) {
    if (x.dtype() != weights.dtype()) {
        DType t = type_promotion(x, weights);
        x = astype(x, t);
        weights = astype(weights, t);
    }
    DALI_ASSERT(x.ndim() == weights.ndim() && x.ndim() >= 1, "circular_convolution: content and weights must have the same (non-zero) number of dimensions");
    std::vector<int> shape = common_shape(x, weights);
    // both operands are presented at the common shape (a broadcast operand is written out once)
    Array xb = x.shape() == shape ? x : identity(broadcasted_reshape(x, shape));
    Array wb = weights.shape() == shape ? weights : identity(broadcasted_reshape(weights, shape));
    return make_node(Kind::CIRCULAR_CONV, "", {xb, wb}, shape, x.dtype());
}

// dali/array/op/concatenate.cpp:9-73: the arrays written one after the other along `axis` into one new buffer
// (dimensions of extent 1 on the other axes are broadcast; the result takes the first array's dtype)
Array concatenate(const std::vector<Array>& arrays, int axis) {
    DALI_ASSERT(!arrays.empty(), "concatenate must receive at least one array.");
    if (arrays.size() == 1) return arrays[0];
    const int nd = arrays[0].ndim();
    DALI_ASSERT(nd > 0, make_message("cannot concatenate scalar arrays (got ndim = ", nd, ")."));
    if (axis < 0) axis += nd;
    DALI_ASSERT(axis >= 0 && axis < nd, make_message("concatenation axis must be >= 0 and < arrays[0].ndim = ", nd, ", but got axis = ", axis, "."));
    std::vector<int> common = arrays[0].shape();
    int total = 0;
    for (const Array& a : arrays) {
        DALI_ASSERT(a.ndim() == nd, make_message("All arrays in concatenate must have the same dimensionality, but got ndim = ", a.ndim(), " != ", nd, "."));
        for (int i = 0; i < nd; ++i) {
            if (i == axis) continue;
            if (common[i] != a.shape()[i] && common[i] == 1) common[i] = a.shape()[i];
            DALI_ASSERT(common[i] == a.shape()[i] || a.shape()[i] == 1,
                        make_message("All shapes must have length-1 or equal dimensions on all axes except the concatenation axis, but got shape ",
                                     shape_str(a.shape()), " which differs on axis ", i, " from expected = ", common[i], "."));
        }
        total += a.shape()[axis];
    }
    std::vector<int> shape = common;
    shape[axis] = total;
    Array result(shape, arrays[0].dtype());
    int so_far = 0;
    for (Array a : arrays) {
        const int n = a.shape()[axis];
        if (n == 0) continue;
        common[axis] = n;
        if (a.dtype() != result.dtype()) a = astype(a, result.dtype());
        if (a.shape() != common) a = broadcasted_reshape(a, common);
        result.slice(axis, so_far, so_far + n).assign(a);
        so_far += n;
    }
    return result;
}
Array hstack(const std::vector<Array>& arrays) { return concatenate(arrays, -1); }
Array vstack(const std::vector<Array>& arrays) { return concatenate(arrays, 0); }

// ---------------------------------------------------------------- sliding windows
// dali/array/op/spatial_utils.cpp:33-50
void check_data_format(const std::string& data_format, int* n_dim, int* c_dim, int* h_dim, int* w_dim) {
    DALI_ASSERT(data_format.size() == 4, make_message("data_format should be a 4 character string containing the letters N, C, H and W (got ",
                                                      data_format, ")."));
    const char letters[4] = {'N', 'C', 'H', 'W'};
    int* outs[4] = {n_dim, c_dim, h_dim, w_dim};
    for (int k = 0; k < 4; ++k) {
        size_t pos = data_format.find(letters[k]);
        DALI_ASSERT(pos != std::string::npos, make_message("data_format should contain character '", letters[k], "' (got ", data_format, ")."));
        *outs[k] = (int)pos;
    }
}

static int int_ceil(int numerator, int denominator) { return (numerator + denominator - 1) / denominator; }

// dali/array/op/spatial_utils.cpp:52-91
template <typename Info>
static Info sliding_window_info(const std::vector<int>& input_shape, int window_h, int window_w, int stride_h, int stride_w, PADDING_T padding,
                                const std::string& data_format) {
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    DALI_ASSERT(input_shape.size() == 4, make_message("sliding-window geometry needs a 4 dimensional shape (got ", shape_str(input_shape), ")."));
    DALI_ASSERT(stride_h > 0 && stride_w > 0, make_message("strides must be strictly positive (got stride_h=", stride_h, ", stride_w=", stride_w, ")."));
    DALI_ASSERT(padding == PADDING_T_SAME || padding == PADDING_T_VALID, make_message("expected padding to be SAME or VALID (got ", (int)padding, ")."));
    Info info;
    info.batch_size = input_shape[n_dim];
    info.in_channels = input_shape[c_dim];
    info.in_h = input_shape[h_dim];
    info.in_w = input_shape[w_dim];
    if (padding == PADDING_T_SAME) {
        info.out_h = int_ceil(info.in_h, stride_h);
        info.out_w = int_ceil(info.in_w, stride_w);
        info.padding_h = std::max(0, (info.out_h - 1) * stride_h + window_h - info.in_h);
        info.padding_w = std::max(0, (info.out_w - 1) * stride_w + window_w - info.in_w);
    } else {
        info.out_h = int_ceil(info.in_h - window_h + 1, stride_h);
        info.out_w = int_ceil(info.in_w - window_w + 1, stride_w);
        info.padding_h = 0;
        info.padding_w = 0;
    }
    info.odd_padding_h = info.padding_h % 2;
    info.odd_padding_w = info.padding_w % 2;
    info.padding_h /= 2;
    info.padding_w /= 2;
    info.stride_h = stride_h;
    info.stride_w = stride_w;
    return info;
}

PoolFunctionInfo compute_pool_info(const std::vector<int>& input_shape, int window_h, int window_w, int stride_h, int stride_w,
                                   PADDING_T padding, const std::string& data_format) {
    PoolFunctionInfo info = sliding_window_info<PoolFunctionInfo>(input_shape, window_h, window_w, stride_h, stride_w, padding, data_format);
    info.window_h = window_h;
    info.window_w = window_w;
    return info;
}

// dali/array/op/spatial_utils.cpp:110-131
ConvFunctionInfo compute_conv2d_info(const std::vector<int>& input_shape, const std::vector<int>& filters_shape, int stride_h,
                                     int stride_w, PADDING_T padding, const std::string& data_format) {
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    DALI_ASSERT(filters_shape.size() == 4, make_message("filters must be 4 dimensional (got ", shape_str(filters_shape), ")."));
    const int filter_h = filters_shape[h_dim], filter_w = filters_shape[w_dim];
    ConvFunctionInfo info = sliding_window_info<ConvFunctionInfo>(input_shape, filter_h, filter_w, stride_h, stride_w, padding, data_format);
    DALI_ASSERT(info.in_channels == filters_shape[c_dim],
                make_message("conv2d input and filters need to have the same number of input channels (got filters input channels = ",
                             filters_shape[c_dim], ", and image input channels = ", info.in_channels, ")."));
    info.filter_h = filter_h;
    info.filter_w = filter_w;
    info.out_channels = filters_shape[n_dim];
    return info;
}

// a 3-D image has no N dimension: the positions of the other letters close up
static std::vector<int> with_batch_axis(const std::vector<int>& shape, int n_dim) {
    std::vector<int> s = shape;
    if (s.size() == 3) s.insert(s.begin() + n_dim, 1);
    return s;
}

// dali/array/op/im2col.cpp:151-188
std::vector<int> im2col_shape(const std::vector<int>& src_shape, int filter_h, int filter_w, int stride_h, int stride_w, int dilate_h,
                              int dilate_w, int prepad_h, int prepad_w, int postpad_h, int postpad_w, const std::string& data_format) {
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    const std::vector<int> s = with_batch_axis(src_shape, n_dim);
    const int i_height = s[h_dim] + prepad_h + postpad_h, i_width = s[w_dim] + prepad_w + postpad_w;
    const int o_height = (i_height - (dilate_h * (filter_h - 1) + 1)) / stride_h + 1;
    const int o_width = (i_width - (dilate_w * (filter_w - 1) + 1)) / stride_w + 1;
    return {filter_h * filter_w * s[c_dim], o_height * o_width * s[n_dim]};
}

// dali/array/op/im2col.cpp:190-267
Array im2col(const Array& image_in, int filter_h, int filter_w, int stride_h, int stride_w, int padding_h, int padding_w, int postpad_h,
             int postpad_w, const std::string& data_format) {
    const int image_ndim = image_in.ndim();
    DALI_ASSERT(image_ndim == 3 || image_ndim == 4, make_message("im2col takes an image with ndim == 3 or ndim == 4 (got ndim=", image_ndim, ")."));
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    Array image = image_ndim == 3 ? image_in.expand_dims(n_dim) : image_in;
    const int image_h = image.shape()[h_dim], image_w = image.shape()[w_dim];
    DALI_ASSERT(image_w >= filter_w && image_h >= filter_h,
                make_message("the image of im2col with data_format=", data_format, " should not be smaller than the filter (filter_h=", filter_h,
                             " vs. image_h=", image_h, ", filter_w=", filter_w, " vs. image_w=", image_w, ")."));
    DALI_ASSERT(filter_h > 0 && filter_w > 0 && stride_h > 0 && stride_w > 0, "im2col: filter sizes and strides must be strictly positive.");
    DALI_ASSERT(padding_h >= 0, make_message("padding_h should be a positive value (got ", padding_h, ")."));
    DALI_ASSERT(padding_w >= 0, make_message("padding_w should be a positive value (got ", padding_w, ")."));
    DALI_ASSERT(postpad_h >= 0, make_message("postpad_h should be a positive value (got ", postpad_h, ")."));
    DALI_ASSERT(postpad_w >= 0, make_message("postpad_w should be a positive value (got ", postpad_w, ")."));
    const int dilate_h = 1, dilate_w = 1;
    Array out = make_node(Kind::IM2COL, "", {image},
                          im2col_shape(image.shape(), filter_h, filter_w, stride_h, stride_w, dilate_h, dilate_w, padding_h, padding_w,
                                       postpad_h, postpad_w, data_format),
                          image.dtype());
    out.expression()->geom = {filter_h, filter_w, stride_h, stride_w, dilate_h, dilate_w, padding_h, padding_w, postpad_h, postpad_w};
    out.expression()->data_format = data_format;
    return out;
}

// dali/array/op/col2im.cpp:165-233
Array col2im(const Array& input, const std::vector<int>& image_shape_in, int filter_h, int filter_w, int stride_h, int stride_w,
             const std::string& data_format) {
    DALI_ASSERT(input.ndim() == 2, make_message("col2im takes a 2D input (got ", input.ndim(), ")."));
    const int image_ndim = (int)image_shape_in.size();
    DALI_ASSERT(image_ndim == 3 || image_ndim == 4, make_message("col2im's image_shape should have size == 3 or 4 (got ", shape_str(image_shape_in), ")."));
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    const std::vector<int> image_shape = with_batch_axis(image_shape_in, n_dim);
    const int image_h = image_shape[h_dim], image_w = image_shape[w_dim], channels = image_shape[c_dim], batch = image_shape[n_dim];
    DALI_ASSERT(filter_h > 0 && filter_w > 0 && stride_h > 0 && stride_w > 0, "col2im: filter sizes and strides must be strictly positive.");
    DALI_ASSERT(image_w >= filter_w && image_h >= filter_h,
                make_message("the image shape of col2im with data_format=", data_format, " should not be smaller than the filter (filter_h=",
                             filter_h, " vs. image_h=", image_h, ", filter_w=", filter_w, " vs. image_w=", image_w, ")."));
    DALI_ASSERT(filter_h * filter_w * channels == input.shape()[0],
                make_message("col2im with data_format ", data_format, "'s input must have its first dimension be filter_h * filter_w * i_channel = ",
                             filter_h * filter_w * channels, " (got ", input.shape()[0], ")."));
    const int o_height = (image_h - filter_h) / stride_h + 1, o_width = (image_w - filter_w) / stride_w + 1;
    DALI_ASSERT(o_height * o_width * batch == input.shape()[1],
                make_message("col2im with data_format ", data_format, "'s input must have its second dimension be ", o_height * o_width * batch,
                             " = out_h [", o_height, "] * out_w [", o_width, "] * batch_size [", batch, "] (got ", input.shape()[1], ")."));
    Array out = make_node(Kind::COL2IM, "", {input}, image_shape, input.dtype());
    out.expression()->geom = {filter_h, filter_w, stride_h, stride_w, 1, 1, 0, 0, 0, 0};
    out.expression()->data_format = data_format;
    // the 4-D form is what the kernel fills; a 3-D request is that buffer without its batch axis
    return image_ndim == 3 ? out.squeeze(n_dim) : out;
}

static void check_nchw_or_nhwc(const char* name, const std::string& data_format) {
    DALI_ASSERT(data_format == "NCHW" || data_format == "NHWC", make_message(name, "'s data_format must be NCHW or NHWC but got ", data_format, " instead."));
}

static void check_ndim4(const char* name, const char* array_name, const Array& a) {
    DALI_ASSERT(a.ndim() == 4, make_message(name, "'s ", array_name, " must be 4 dimensional but got ", array_name, " with ndim = ", a.ndim(), "."));
}

// dali/array/op/conv.cpp:223-276: filters [out, ...] flattened to a matrix times the patch matrix
Array conv2d(const Array& input, const Array& filters, int stride_h, int stride_w, PADDING_T padding, const std::string& data_format) {
    DALI_ASSERT(input.ndim() == 3 || input.ndim() == 4, make_message("Input argument to conv2d must be 3D or 4D (got input.ndim=", input.ndim(), ")."));
    check_ndim4("conv2d", "filters", filters);
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    check_nchw_or_nhwc("conv2d", data_format);
    ConvFunctionInfo info = compute_conv2d_info(with_batch_axis(input.shape(), n_dim), filters.shape(), stride_h, stride_w, padding, data_format);
    // channels-last, stride 1: no patch matrix (see conv2d_direct_nhwc); DALI_HIP_CONV_IM2COL=1 keeps the two-step form
    static const bool two_step = getenv("DALI_HIP_CONV_IM2COL") != nullptr;
    if (!two_step && !dry_run() && data_format == "NHWC" && stride_h == 1 && stride_w == 1 && input.ndim() == 4 && input.dtype() == DTYPE_FLOAT &&
        filters.dtype() == DTYPE_FLOAT && info.in_channels % 4 == 0 && info.filter_h <= 8 &&
        (int64_t)info.batch_size * (info.in_h + 2 * info.padding_h + info.odd_padding_h + info.filter_h) *
                (info.in_w + 2 * info.padding_w + info.odd_padding_w + info.filter_w) * info.in_channels < ((int64_t)1 << 30)) {
        input.eval();
        filters.eval();
        return conv2d_direct_nhwc(input, filters, info.padding_h, info.padding_w, info.padding_h + info.odd_padding_h,
                                  info.padding_w + info.odd_padding_w);
    }
    Array filters_nxxx = filters.swapaxes(n_dim, 0);
    Array filters_nX = filters_nxxx.reshape({filters_nxxx.shape()[0], -1});
    Array patches = im2col(input, info.filter_h, info.filter_w, stride_h, stride_w, info.padding_h, info.padding_w,
                           info.padding_h + info.odd_padding_h, info.padding_w + info.odd_padding_w, data_format);
    if (data_format == "NCHW")
        return dot(filters_nX, patches).reshape({info.out_channels, info.batch_size, info.out_h, info.out_w}).swapaxes(0, 1);
    // the filter matrix is written out transposed (a few hundred KB): the product then reads both operands along their rows
    return dot(patches.transpose(), filters_nX.transpose().ascontiguousarray()).reshape({info.batch_size, info.out_h, info.out_w, info.out_channels});
}

// dali/array/op/conv.cpp:278-336. The adjoint of im2col takes no padding (col2im.cpp:217-232), so, like the
// reference, this is defined for convolutions whose windows tile the image without padding.
Array conv2d_backward_input(Array filters, Array out_dw, int stride_h, int stride_w, const std::vector<int>& result_shape, PADDING_T padding,
                            const std::string& data_format) {
    check_ndim4("conv2d_backward_input", "out_dw", out_dw);
    check_ndim4("conv2d_backward_input", "filters", filters);
    check_nchw_or_nhwc("conv2d_backward_input", data_format);
    DALI_ASSERT(result_shape.size() == 4, make_message("conv2d_backward_input's result_shape must be of size 4, but got ", shape_str(result_shape), "."));
    ConvFunctionInfo info = compute_conv2d_info(result_shape, filters.shape(), stride_h, stride_w, padding, data_format);
    Array filters2d = filters.reshape({filters.shape()[0], -1});  // [out, filter_h * filter_w * in]
    if (data_format == "NCHW") {
        Array out_dw_cnhw = out_dw.swapaxes(0, 1);
        out_dw_cnhw = out_dw_cnhw.reshape({out_dw_cnhw.shape()[0], -1});
        return col2im(dot(filters2d.transpose(), out_dw_cnhw), result_shape, info.filter_h, info.filter_w, stride_h, stride_w, data_format);
    }
    // NHWC: the patch-matrix gradient Filters^T . dOut^T is formed patch-major, as [N*h*w, window*c] = dOut . Filters, and handed
    // over as its transposed view: the same numbers, laid out so that the channel run of a pixel is contiguous
    Array out_dw2d = out_dw.reshape({-1, out_dw.shape()[3]});  // [N*h*w, out]
    return col2im(dot(out_dw2d, filters2d).transpose(), result_shape, info.filter_h, info.filter_w, stride_h, stride_w, data_format);
}

// dali/array/op/conv.cpp:338-393
Array conv2d_backward_filters(Array input, Array out_dw, int stride_h, int stride_w, const std::vector<int>& filters_shape, PADDING_T padding,
                              const std::string& data_format) {
    check_ndim4("conv2d_backward_filters", "out_dw", out_dw);
    check_ndim4("conv2d_backward_filters", "input", input);
    check_nchw_or_nhwc("conv2d_backward_filters", data_format);
    DALI_ASSERT(filters_shape.size() == 4, make_message("conv2d_backward_filters's filters_shape must be of size 4, but got ", shape_str(filters_shape), "."));
    ConvFunctionInfo info = compute_conv2d_info(input.shape(), filters_shape, stride_h, stride_w, padding, data_format);
    Array patches_t = im2col(input, info.filter_h, info.filter_w, stride_h, stride_w, info.padding_h, info.padding_w,
                             info.padding_h + info.odd_padding_h, info.padding_w + info.odd_padding_w, data_format).transpose();
    if (data_format == "NCHW") {
        Array out_dw_cnhw = out_dw.swapaxes(1, 0);
        out_dw_cnhw = out_dw_cnhw.reshape({out_dw_cnhw.shape()[0], -1});
        return dot(out_dw_cnhw, patches_t).reshape(filters_shape);
    }
    out_dw = out_dw.reshape({-1, out_dw.shape()[3]}).transpose();
    return dot(out_dw, patches_t).reshape(filters_shape);
}

// dali/array/op/conv.cpp:395-401
Array conv2d_backward_bias(Array out_dw, const std::string& data_format) {
    check_ndim4("conv2d_backward_bias", "out_dw", out_dw);
    int n_dim, c_dim, h_dim, w_dim;
    check_data_format(data_format, &n_dim, &c_dim, &h_dim, &w_dim);
    return sum(out_dw, {n_dim, h_dim, w_dim});
}

// dali/array/op/conv.cpp:403-428
Array pool2d(const Array& input, int window_h, int window_w, int stride_h, int stride_w, POOLING_T pooling_mode, PADDING_T padding,
             const std::string& data_format) {
    check_ndim4("pool2d", "input", input);
    check_nchw_or_nhwc("pool2d", data_format);
    DALI_ASSERT(window_h > 0 && window_w > 0, make_message("pool2d windows must be strictly positive (got ", window_h, " x ", window_w, ")."));
    PoolFunctionInfo info = compute_pool_info(input.shape(), window_h, window_w, stride_h, stride_w, padding, data_format);
    const bool nchw = data_format == "NCHW";
    std::vector<int> shape = nchw ? std::vector<int>{info.batch_size, info.in_channels, info.out_h, info.out_w}
                                  : std::vector<int>{info.batch_size, info.out_h, info.out_w, info.in_channels};
    Array out = make_node(Kind::POOL2D, pooling_mode == POOLING_T_MAX ? "reducers::maximum" : "reducers::avg", {input}, shape, input.dtype());
    out.expression()->geom = {info.window_h, info.window_w, info.stride_h, info.stride_w, info.padding_h, info.padding_w};
    out.expression()->data_format = data_format;
    out.expression()->depth = pooling_mode == POOLING_T_AVG ? 1 : 0;
    return out;
}

// dali/array/op/conv.cpp:430-456
Array pool2d_backward(const Array& y, const Array& dy, const Array& x, int window_h, int window_w, int stride_h, int stride_w,
                      POOLING_T pooling_mode, PADDING_T padding, const std::string& data_format) {
    check_ndim4("pool2d_backward", "y", y);
    check_ndim4("pool2d_backward", "dy", dy);
    check_ndim4("pool2d_backward", "x", x);
    check_nchw_or_nhwc("pool2d_backward", data_format);
    PoolFunctionInfo info = compute_pool_info(x.shape(), window_h, window_w, stride_h, stride_w, padding, data_format);
    DALI_ASSERT(y.shape() == dy.shape(), make_message("pool2d_backward: y ", shape_str(y.shape()), " and dy ", shape_str(dy.shape()), " must have the same shape."));
    DALI_ASSERT(y.dtype() == dy.dtype() && y.dtype() == x.dtype(), "pool2d_backward: y, dy and x must have the same dtype.");
    Array out = make_node(Kind::POOL2D_BACKWARD, pooling_mode == POOLING_T_MAX ? "reducers::maximum" : "reducers::avg", {y, dy, x}, x.shape(), y.dtype());
    out.expression()->geom = {info.window_h, info.window_w, info.stride_h, info.stride_w, info.padding_h, info.padding_w};
    out.expression()->data_format = data_format;
    out.expression()->depth = pooling_mode == POOLING_T_AVG ? 1 : 0;
    return out;
}

// dali/array/op/one_hot.cpp:62-74
Array one_hot(Array indices, int depth, Array on_value, Array off_value) {
    DALI_ASSERT(indices.dtype() == DTYPE_INT32, "indices must be integers.");
    DALI_ASSERT(on_value.is_scalar(), make_message("on_value must be a scalar (got on_value.ndim=", on_value.ndim(), ")."));
    DALI_ASSERT(off_value.is_scalar(), make_message("off_value must be a scalar (got off_value.ndim=", off_value.ndim(), ")."));
    DALI_ASSERT(depth > 0, make_message("depth must be strictly positive (got depth=", depth, ")."));
    if (on_value.dtype() != off_value.dtype()) {
        DType t = type_promotion(on_value, off_value);
        on_value = astype(on_value, t);
        off_value = astype(off_value, t);
    }
    std::vector<int> shape = indices.shape();
    shape.push_back(depth);
    auto out = make_node(Kind::ONE_HOT, "", {on_value, off_value, indices}, shape, on_value.dtype());
    out.expression()->depth = depth;
    return out;
}

// dali/array/op/dot.cpp:49-67
Array matmul(Array a, Array b) {
    DALI_ASSERT(a.ndim() == 2 && b.ndim() == 2,
                make_message("matmul inputs must be both be 2-dimensional, but got a.ndim = ", a.ndim(), " and b.ndim = ", b.ndim(), "."));
    DALI_ASSERT(a.shape()[1] == b.shape()[0] || a.shape()[1] == 1 || b.shape()[0] == 1,
                make_message("matmul shapes not aligned, with a.shape = ", shape_str(a.shape()), " and b.shape = ", shape_str(b.shape()),
                             ": expected a.shape[1] = ", a.shape()[1], " to equal b.shape[0] = ", b.shape()[0], ", or for either to equal 1."));
    if (a.shape()[1] != b.shape()[0]) {
        if (a.shape()[1] == 1)
            a = broadcasted_reshape(a, {a.shape()[0], b.shape()[0]});
        else
            b = broadcasted_reshape(b, {a.shape()[1], b.shape()[1]});
    }
    DType t = type_promotion(a, b);
    if (a.dtype() != t) a = astype(a, t);
    if (b.dtype() != t) b = astype(b, t);
    return make_node(Kind::MATMUL, "", {a, b}, {a.shape()[0], b.shape()[1]}, t);
}

// A [rows, cols] matrix made of `x` with its axes taken in the order `order`, the first `lead` of them forming the rows.
// Dense buffers whose order is the identity or a rotation become a view (the rotation is a transposed matrix, which the
// GEMM reads in place); any other order is written out once.
static Array as_matrix(const Array& x, const std::vector<int>& order, int lead) {
    const int nd = x.ndim();
    int64_t rows = 1, cols = 1;
    for (int i = 0; i < nd; ++i) (i < lead ? rows : cols) *= x.shape()[order[i]];
    DALI_ASSERT(rows <= std::numeric_limits<int>::max() && cols <= std::numeric_limits<int>::max(), "tensordot: operand too large");
    bool identity = true, rotation = true;
    for (int i = 0; i < nd; ++i) {
        identity = identity && order[i] == i;
        rotation = rotation && order[i] == (i + (nd - lead)) % nd;
    }
    if (identity) return x.reshape({(int)rows, (int)cols});
    if (rotation && x.is_buffer() && x.contiguous_memory()) return x.reshape({(int)cols, (int)rows}).transpose();
    return x.transpose(order).reshape({(int)rows, (int)cols});
}

static void check_tensordot_axes(const Array& x, char name, std::vector<int>& axes) {
    const int nd = x.ndim();
    DALI_ASSERT((int)axes.size() <= nd, make_message("tensordot's length of argument ", name, "_reduce_axes should be less than the dimensions of ",
                                                     name, " (", name, ".ndim = ", nd, ", ", name, "_reduce_axes.size() = ", axes.size(), ")."));
    std::vector<bool> seen(nd, false);
    for (int& ax : axes) {
        if (ax < 0) ax += nd;
        DALI_ASSERT(ax >= 0 && ax < nd, make_message(name, "_reduce_axes contains reduction dimensions that are greater than or equal to ", name,
                                                     ".ndim (", name, ".ndim = ", nd, ", and found ", ax, ")."));
        DALI_ASSERT(!seen[ax], make_message("tensordot: axis ", ax, " of ", name, " is named twice."));
        seen[ax] = true;
    }
}

// dali/array/gemm/tensordot_as_dot.h:120-158: the kept axes of a, then its reduced axes, against the reduced axes of b,
// then its kept ones; one matrix product; the result has the kept axes of a followed by those of b.
Array tensordot(const Array& a, const Array& b, const std::vector<int>& a_reduce_axes, const std::vector<int>& b_reduce_axes) {
    DALI_ASSERT(a_reduce_axes.size() == b_reduce_axes.size(),
                make_message("tensordot_as_dot must have as many reduction axes for a than b (got a_reduce_axes.size() = ", a_reduce_axes.size(),
                             " and b_reduce_axes.size() = ", b_reduce_axes.size(), ")."));
    std::vector<int> ra = a_reduce_axes, rb = b_reduce_axes;
    check_tensordot_axes(a, 'a', ra);
    check_tensordot_axes(b, 'b', rb);
    std::vector<int> order_a, order_b = rb, out_shape;
    for (int i = 0; i < a.ndim(); ++i)
        if (std::find(ra.begin(), ra.end(), i) == ra.end()) {
            order_a.push_back(i);
            out_shape.push_back(a.shape()[i]);
        }
    const int kept_a = (int)order_a.size();
    order_a.insert(order_a.end(), ra.begin(), ra.end());
    for (int i = 0; i < b.ndim(); ++i)
        if (std::find(rb.begin(), rb.end(), i) == rb.end()) {
            order_b.push_back(i);
            out_shape.push_back(b.shape()[i]);
        }
    for (size_t i = 0; i < ra.size(); ++i)
        DALI_ASSERT(a.shape()[ra[i]] == b.shape()[rb[i]],
                    make_message("tensordot shapes not aligned, with a.shape = ", shape_str(a.shape()), " and b.shape = ", shape_str(b.shape()),
                                 ": a.shape[", ra[i], "] = ", a.shape()[ra[i]], " != b.shape[", rb[i], "] = ", b.shape()[rb[i]], "."));
    return matmul(as_matrix(a, order_a, kept_a), as_matrix(b, order_b, (int)rb.size())).reshape(out_shape);
}

// dali/array/gemm/tensordot_as_dot.h:48-118: the last `axis` axes of a against the first `axis` axes of b
Array tensordot(const Array& a, const Array& b, int axis) {
    DALI_ASSERT(axis >= 0, make_message("tensordot_as_dot axis must be a non-negative integer (got axis = ", axis, ")."));
    DALI_ASSERT(axis <= a.ndim(), make_message("tensordot_as_dot axis can not be larger than the dimension of a (a.ndim() = ", a.ndim(), ", axis = ", axis, ")."));
    DALI_ASSERT(axis <= b.ndim(), make_message("tensordot_as_dot axis can not be larger than the dimension of b (b.ndim() = ", b.ndim(), ", axis = ", axis, ")."));
    std::vector<int> ra, rb;
    for (int i = 0; i < axis; ++i) {
        ra.push_back(a.ndim() - axis + i);
        rb.push_back(i);
    }
    return tensordot(a, b, ra, rb);
}

// dali/array/op/top_k.cpp:198-233. The reference computes these on the CPU only; here the rows are ordered on the
// device. Unlike the other factories these evaluate their argument at once.
static Array k_best(const Array& array, int k, bool largest, const char* name) {
    DALI_ASSERT(k >= 1, make_message(name, "'s k argument must be >= 1, but got k = ", k, "."));
    if (array.number_of_elements() == 1) return Array::zeros(array.shape(), DTYPE_INT32);
    DALI_ASSERT(array.ndim() >= 1, make_message(name, " expects an array with at least one dimension."));
    const int cols = array.shape().back();
    DALI_ASSERT(k <= cols, make_message(name, "'s k argument must be <= the last dimension (got k = ", k, ", shape = ", shape_str(array.shape()), ")."));
    if (k == 1) return (largest ? argmax(array, -1) : argmin(array, -1)).expand_dims(-1);
    std::vector<int> shape = array.shape();
    shape.back() = k;
    // the reference's heap breaks ties of bottom_k towards the higher column (top_k.cpp:118-123), its full sort
    // (k = the whole row) towards the lower one (top_k.cpp:139-158)
    return topk_rows(array.reshape({-1, cols}), k, largest, !largest && k < cols).reshape(shape);
}
Array top_k(const Array& array, int k, bool sorted) {
    (void)sorted;  // the unsorted form promises no order; the sorted one is returned for both
    return k_best(array, k, true, "top_k");
}
Array bottom_k(const Array& array, int k, bool sorted) {
    (void)sorted;
    return k_best(array, k, false, "bottom_k");
}
Array argsort(const Array& array) {
    Array raveled = array.reshape({-1});
    return bottom_k(raveled, raveled.number_of_elements(), true);
}
Array argsort(const Array& array, int axis) {
    if (array.ndim() == 0) return Array::zeros({}, DTYPE_INT32);
    if (axis < 0) axis += array.ndim();
    DALI_ASSERT(axis >= 0 && axis < array.ndim(), make_message("argsort axis must >= 0 and < ndim (", array.ndim(), "), got axis = ", axis, "."));
    return bottom_k(array.swapaxes(axis, -1), array.shape()[axis], true).swapaxes(axis, -1);
}

// dali/array/op/dot.cpp:100-102
Array inner(const Array& a, const Array& b) {
    DALI_ASSERT(a.ndim() == 1 && b.ndim() == 1,
                make_message("inner expects vector inputs but got a.ndim = ", a.ndim(), " and b.ndim = ", b.ndim(), " arrays."));
    DALI_ASSERT(a.shape()[0] == b.shape()[0], make_message("inner input shapes a.shape = ", shape_str(a.shape()),
                                                           " and b.shape = ", shape_str(b.shape()), " should be equal."));
    return matmul(a.reshape({1, a.number_of_elements()}), b.reshape({b.number_of_elements(), 1})).reshape({});
}

// dali/array/op/dot.cpp:67-90
Array matrix_vector_dot(const Array& a, const Array& b) {
    DALI_ASSERT((a.ndim() == 1 && b.ndim() == 2) || (a.ndim() == 2 && b.ndim() == 1),
                make_message("matrix_vector_dot inputs must be a vector and a matrix, but got a.ndim = ", a.ndim(), " and b.ndim = ", b.ndim(), "."));
    if (a.ndim() == 1) {
        DALI_ASSERT(b.shape()[0] == a.shape()[0], make_message("matrix_vector_dot shape mistmach between a.shape = ", shape_str(a.shape()),
                                                               " and b.shape = ", shape_str(b.shape()), "."));
        return matmul(a.reshape({1, a.number_of_elements()}), b).reshape({b.shape()[1]});
    }
    DALI_ASSERT(a.shape()[1] == b.shape()[0], make_message("matrix_vector_dot shape mistmach between a.shape = ", shape_str(a.shape()),
                                                           " and b.shape = ", shape_str(b.shape()), "."));
    return matmul(a, b.reshape({b.number_of_elements(), 1})).reshape({a.shape()[0]});
}

// dali/array/op/dot.cpp:104-124
Array dot(const Array& a, const Array& b) {
    int an = a.ndim(), bn = b.ndim();
    if (an == 0 || bn == 0) return eltmul(a, b);
    // a is reduced over its last axis, b over its second to last one (its only one when it is a vector)
    if (an > 2 || bn > 2) return tensordot(a, b, std::vector<int>{an - 1}, std::vector<int>{std::max(0, bn - 2)});
    if (an == 1 && bn == 1) return inner(a, b);
    if (an == 2 && bn == 2) return matmul(a, b);
    return matrix_vector_dot(a, b);
}

CrossEntropyResult softmax_cross_entropy(const Array& logits, const Array& targets) {
    DALI_ASSERT(logits.ndim() == 2, "softmax_cross_entropy expects 2-D logits");
    DALI_ASSERT(targets.ndim() == 1 && targets.dtype() == DTYPE_INT32 && targets.shape()[0] == logits.shape()[0],
                "softmax_cross_entropy expects one int32 target per row");
    int rows = logits.shape()[0], cols = logits.shape()[1];
    {
        // Rows that are few for their length: one launch would give each row to one workgroup, which streams it through a single
        // compute unit three times ([7,9999999]: 3.5 ms). The statistics come from pieces of the rows instead, and gradient and
        // losses are then maps over them: the logits are read twice and nothing else is as large.
        Array x = logits, M, L;
        if (!dry_run() && few_long_rows_softmax_statistics(&x, &M, &L)) {
            Array grad = subtract(eltdiv(exp(subtract(x, M)), L), one_hot(targets, cols, Array(1.0f), Array(0.0f)));
            Array row_loss = subtract(add(log(L), M), gather_from_rows(x, targets).expand_dims(1));
            Array mean_loss = mean(row_loss);
            grad.eval();
            Array::eval_together({row_loss, mean_loss});
            return {mean_loss, row_loss.reshape({rows}), grad};
        }
    }
    Array m = max(logits, {-1}, true);
    Array exped = exp(subtract(logits, m));
    Array s = sum(exped, {-1}, true);
    Array grad = subtract(eltdiv(exped, s), one_hot(targets, cols, Array(1.0f), Array(0.0f)));
    // lse = log(s) + m, shape [rows, 1]; row loss = lse - logits[i, t_i]
    Array lse = add(log(s), m);
    Array picked = gather_from_rows(logits, targets).expand_dims(1);
    Array row_loss = subtract(lse, picked);
    // the mean over the rows rides along in the same launch (its partial sums meet in the library workspace)
    Array mean_loss = mean(row_loss);
    Array::eval_together({grad, row_loss, mean_loss});
    Array rows1d = row_loss.reshape({rows});
    return {mean_loss, rows1d, grad};
}

// Whether the recurrent half of a sequence goes into one persistent launch: where the library expects that to beat a launch per
// step of the fused step (answer 2); where the fused step does not apply (an input or hidden size that is no multiple of 64: two products and a gate
// kernel per step), wherever it is served up to the batch it was measured to win at against that form; `always`: wherever served.
static bool persistent_wins(int Bn, int In, int H, bool always) {
    const int served = dali_hip_lstm_recurrent_persistent_supported(Bn, H);
    if (always) return served >= 1;
    const bool fused_applies = H % 64 == 0 && In % 64 == 0;
    return served == 2 || (served == 1 && !fused_applies && Bn <= 96);
}

LSTMState lstm_step(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U, const Array& b) {
    DALI_ASSERT(x.ndim() == 2 && h.ndim() == 2 && c.ndim() == 2 && W.ndim() == 2 && U.ndim() == 2 && b.ndim() == 1,
                "lstm_step: x, h, c, W, U must be matrices and b a vector");
    int H = h.shape()[1];
    DALI_ASSERT(W.shape()[1] == 4 * H && U.shape()[1] == 4 * H && b.shape()[0] == 4 * H && U.shape()[0] == H &&
                    W.shape()[0] == x.shape()[1] && c.shape() == h.shape() && x.shape()[0] == h.shape()[0],
                "lstm_step: inconsistent shapes");
    // one launch when the fused kernel applies: the gate arithmetic runs in the GEMM's epilogue
    static const bool fused_off = getenv("DALI_HIP_LSTM_UNFUSED") != nullptr;
    const int Bn = x.shape()[0], In = x.shape()[1];
    auto dense = [](const Array& a) { return a.is_buffer() && a.contiguous_memory() && a.dtype() == DTYPE_FLOAT; };
    for (const Array* a : {&x, &h, &c, &W, &U, &b}) a->eval();
    // up to 64 rows: the 64-row tiles of the general kernel would mostly multiply padding (37 us whatever the batch); 16-row
    // tiles with every compute unit on its own columns of the weights
    const char* small_env = getenv("DALI_HIP_LSTM_SMALL");
    const bool small_off = small_env != nullptr && std::string(small_env) == "0";
    // (from 17 rows on, where the fused step applies, that one is faster: its inner extent is cut into one share per compute unit
    // and it takes 17.3-18.8 us for up to 64 rows of 1024, against 18.4-31.0 us here)
    const bool fused_applies = H % 64 == 0 && In % 64 == 0;
    if (!fused_off && !small_off && !dry_run() && Bn <= (fused_applies ? 16 : 64) && H % 256 == 0 && H <= 1024 && In % 16 == 0 && (In + H) % 64 == 0 && dense(x) && dense(h) &&
        dense(c) && dense(W) && dense(U) && dense(b) && x.offset() % 4 == 0 && h.offset() % 4 == 0 && W.offset() % 4 == 0 && U.offset() % 4 == 0 && c.offset() % 4 == 0) {
        Array c_new({Bn, H}, DTYPE_FLOAT), h_new({Bn, H}, DTYPE_FLOAT);
        lstm_step_small(x, h, c, W, U, b, c_new, h_new);
        return {c_new, h_new};
    }
    if (!fused_off && !dry_run() && H % 64 == 0 && In % 64 == 0 && dense(x) && dense(h) && dense(c) && dense(W) && dense(U) && dense(b) &&
        x.offset() % 4 == 0 && h.offset() % 4 == 0 && W.offset() % 4 == 0 && U.offset() % 4 == 0) {
        Array c_new({Bn, H}, DTYPE_FLOAT), h_new({Bn, H}, DTYPE_FLOAT);
        lstm_step_fused(x, h, c, W, U, b, c_new, h_new);
        return {c_new, h_new};
    }
    // pre-activations: one accumulating GEMM pair (X.W + H.U)
    Array pre = add(dot(x, W), dot(h, U));
    pre.eval();
    auto gate = [&](int k) {
        Array bias = b.slice(0, k * H, (k + 1) * H).expand_dims(0);
        return add(pre.slice(1, k * H, (k + 1) * H), bias);
    };
    Array ig = sigmoid(gate(0)), fg = sigmoid(gate(1)), og = sigmoid(gate(2)), cw = tanh(gate(3));
    Array c_new = add(eltmul(fg, c), eltmul(ig, cw));
    Array h_new = eltmul(og, tanh(c_new));
    Array::eval_together({c_new, h_new});
    return {c_new, h_new};
}

// The step above applied along a sequence (dali/layers/lstm.cpp:294-303): xs is [T, B, I]; returns every hidden
// state as one [T, B, H] buffer plus the final cell state. With the fused kernel each step is one launch that reads
// h(t-1) from, and writes h(t) into, its slice of that buffer; nothing is copied between steps.
LSTMSequence lstm_sequence(const Array& xs, const Array& h0, const Array& c0, const Array& W, const Array& U, const Array& b) {
    DALI_ASSERT(xs.ndim() == 3 && h0.ndim() == 2 && c0.ndim() == 2, "lstm_sequence: xs must be [T, B, I], h0 and c0 [B, H]");
    const int T = xs.shape()[0], Bn = xs.shape()[1], In = xs.shape()[2], H = h0.shape()[1];
    DALI_ASSERT(T >= 1, "lstm_sequence: the sequence must hold at least one step");
    DALI_ASSERT(h0.shape()[0] == Bn && c0.shape() == h0.shape(), "lstm_sequence: inconsistent batch sizes");
    static const bool fused_off = getenv("DALI_HIP_LSTM_UNFUSED") != nullptr;
    auto dense = [](const Array& a) { return a.is_buffer() && a.contiguous_memory() && a.dtype() == DTYPE_FLOAT; };
    for (const Array* a : {&xs, &h0, &c0, &W, &U, &b}) a->eval();
    Array seq = xs.is_buffer() && xs.contiguous_memory() ? xs : xs.ascontiguousarray();
    Array hs({T, Bn, H}, DTYPE_FLOAT);
    Array cells[2] = {Array({Bn, H}, DTYPE_FLOAT), Array({Bn, H}, DTYPE_FLOAT)};
    const bool fused = !fused_off && !dry_run() && H % 64 == 0 && In % 64 == 0 && dense(seq) && dense(h0) && dense(c0) && dense(W) && dense(U) && dense(b) &&
                       W.ndim() == 2 && U.ndim() == 2 && b.ndim() == 1 && W.shape()[0] == In && W.shape()[1] == 4 * H && U.shape()[0] == H &&
                       U.shape()[1] == 4 * H && b.shape()[0] == 4 * H && seq.offset() % 4 == 0 && h0.offset() % 4 == 0 && W.offset() % 4 == 0 &&
                       U.offset() % 4 == 0 && ((int64_t)Bn * H) % 4 == 0;
    // Small batches: a launch per step waits more than it works (37 us per step from 1 to 128 rows). The input half of
    // every step's pre-activations is one product over all T * B rows, and the recurrent half runs as one persistent launch
    // that keeps U on the chip (in the LDS or the registers of the compute units).
    const char* persistent_env = getenv("DALI_HIP_LSTM_PERSISTENT");  // read per call: a benchmark times both forms in one process
    const bool persistent_off = persistent_env != nullptr && std::string(persistent_env) == "0";
    const bool persistent_ok = !persistent_off && !dry_run() && T >= 2 && dense(seq) && dense(h0) && dense(c0) && dense(W) && dense(U) && dense(b) &&
                               W.ndim() == 2 && U.ndim() == 2 && b.ndim() == 1 && W.shape()[0] == In && W.shape()[1] == 4 * H && U.shape()[0] == H &&
                               U.shape()[1] == 4 * H && b.shape()[0] == 4 * H && c0.offset() % 4 == 0 && ((int64_t)Bn * H) % 4 == 0 &&
                               persistent_wins(Bn, In, H, persistent_env != nullptr && std::string(persistent_env) == "2");
    // (a size that the persistent kernels do not serve, or serve more slowly than a launch per step, takes the loop below; a failure of the
    // launch itself is an error)
    if (persistent_ok) {
        Array pre = add(dot(seq.reshape({T * Bn, In}), W), b.expand_dims(0));
        pre.eval();
        Array c_last({Bn, H}, DTYPE_FLOAT);
        Array h0c = h0.offset() % 4 == 0 ? h0 : h0.ascontiguousarray();
        lstm_recurrent_persistent(pre.reshape({T, Bn, 4 * H}), U, h0c, c0, hs, c_last);
        return {hs, c_last, hs[T - 1]};
    }
    Array c_prev = c0, h_prev = h0;
    // Sizes the fused step does not take (a hidden size of 1000): the input half of every step's pre-activations is one product
    // over all T * B rows, bias included; a step is then the recurrent product and one kernel that adds the two halves, applies
    // the gates and writes c(t) and h(t) in place (B = 64, I = H = 1000: 41 -> 19 us per step; three launches a step before,
    // one of them a copy of h(t) into the sequence)
    static const bool batched_off = getenv("DALI_HIP_LSTM_BATCHED_INPUT") != nullptr && std::string(getenv("DALI_HIP_LSTM_BATCHED_INPUT")) == "0";
    if (!fused && !batched_off && !dry_run() && T >= 2 && dense(seq) && dense(h0) && dense(c0) && dense(W) && dense(U) && dense(b) && W.ndim() == 2 && U.ndim() == 2 &&
        b.ndim() == 1 && W.shape()[0] == In && W.shape()[1] == 4 * H && U.shape()[0] == H && U.shape()[1] == 4 * H && b.shape()[0] == 4 * H) {
        Array pre = add(dot(seq.reshape({T * Bn, In}), W), b.expand_dims(0));
        pre.eval();
        Array pre3 = pre.reshape({T, Bn, 4 * H});
        for (int t = 0; t < T; ++t) {
            Array rec = dot(h_prev, U);
            rec.eval();
            Array in_t = pre3[t];
            auto gate = [&](int k) { return add(in_t.slice(1, k * H, (k + 1) * H), rec.slice(1, k * H, (k + 1) * H)); };
            Array ig = sigmoid(gate(0)), fg = sigmoid(gate(1)), og = sigmoid(gate(2)), cw = tanh(gate(3));
            Array c_new = add(eltmul(fg, c_prev), eltmul(ig, cw));
            Array h_new = eltmul(og, tanh(c_new));
            evaluate_into_together({cells[t % 2], hs[t]}, {c_new, h_new});
            c_prev = cells[t % 2];
            h_prev = hs[t];
        }
        return {hs, c_prev, h_prev};
    }
    for (int t = 0; t < T; ++t) {
        Array x_t = seq[t], h_t = hs[t];
        if (fused) {
            lstm_step_fused(x_t, h_prev, c_prev, W, U, b, cells[t % 2], h_t);
            c_prev = cells[t % 2];
        } else {
            LSTMState st = lstm_step(x_t, h_prev, c_prev, W, U, b);
            h_t.assign(st.hidden);
            c_prev = st.memory;
        }
        h_prev = h_t;
    }
    return {hs, c_prev, h_prev};
}

// dali/layers/stacked_lstm.cpp:219-283 with drop_prob = 0. A shortcut layer's two inputs are laid side by side so that
// the layer stays one accumulating GEMM pair plus the gate kernel.
StackedLSTMState stacked_lstm_step(const Array& x, const std::vector<Array>& h, const std::vector<Array>& c, const std::vector<Array>& W,
                                   const std::vector<Array>& U, const std::vector<Array>& b, bool shortcut) {
    const size_t layers = W.size();
    DALI_ASSERT(h.size() == layers && c.size() == layers,
                make_message("Activating LSTM stack of size ", layers, " with different number of states ", std::min(h.size(), c.size())));
    DALI_ASSERT(U.size() == layers && b.size() == layers, "stacked_lstm_step: every layer needs its W, U and b");
    StackedLSTMState out;
    Array layer_input = x;
    for (size_t l = 0; l < layers; ++l) {
        Array in = (shortcut && l > 0) ? concatenate({layer_input, x}, 1) : layer_input;
        LSTMState st = lstm_step(in, h[l], c[l], W[l], U[l], b[l]);
        out.memory.push_back(st.memory);
        out.hidden.push_back(st.hidden);
        layer_input = st.hidden;
    }
    return out;
}

// AbstractStackedLSTM::activate_sequence (dali/layers/stacked_lstm.cpp:44-51, drop_prob = 0): the stack applied to every
// x(t) in turn. Layer l at step t needs layer l-1 at step t and itself at step t-1 only, so the loop nest can be turned
// around: every layer runs over the whole sequence before the next one starts, on the hidden states of the layer below
// ([T, B, H], beside x(t) for a shortcut stack), which lets each layer take the one-launch recurrence of lstm_sequence.
StackedLSTMSequence stacked_lstm_sequence(const Array& xs, const std::vector<Array>& h, const std::vector<Array>& c, const std::vector<Array>& W,
                                          const std::vector<Array>& U, const std::vector<Array>& b, bool shortcut) {
    const size_t layers = W.size();
    DALI_ASSERT(xs.ndim() == 3, "stacked_lstm_sequence: xs must be [T, B, I]");
    DALI_ASSERT(h.size() == layers && c.size() == layers,
                make_message("Activating LSTM stack of size ", layers, " with different number of states ", std::min(h.size(), c.size())));
    DALI_ASSERT(U.size() == layers && b.size() == layers && layers >= 1, "stacked_lstm_sequence: every layer needs its W, U and b");
    StackedLSTMSequence out;
    Array layer_input = xs;
    for (size_t l = 0; l < layers; ++l) {
        Array in = (shortcut && l > 0) ? concatenate({layer_input, xs}, 2) : layer_input;
        LSTMSequence r = lstm_sequence(in, h[l], c[l], W[l], U[l], b[l]);
        out.memory.push_back(r.memory);
        out.hidden.push_back(r.hidden);
        layer_input = r.hidden_states;
    }
    out.top_hidden_states = layer_input;
    return out;
}

// One GRU step (dali/layers/gru.cpp:27-44 with StackedInputLayer::activate, dali/layers/layers.cpp:159-161), the
// three input layers packed reset, update, candidate along the columns of W[I, 3H], U[H, 3H], b[3H]:
//   r = sigmoid(x.Wr + h.Ur + br);  z = sigmoid(x.Wz + h.Uz + bz);  m = tanh(x.Wc + (r * h).Uc + bc)
//   h' = h * (1.0 - z) + m * z
// Three matrix products (the candidate's recurrent product needs r first) and two fused elementwise kernels.
Array gru_step(const Array& x, const Array& h, const Array& W, const Array& U, const Array& b) {
    DALI_ASSERT(x.ndim() == 2 && h.ndim() == 2 && W.ndim() == 2 && U.ndim() == 2 && b.ndim() == 1, "gru_step: x, h, W, U must be matrices and b a vector");
    const int H = h.shape()[1];
    DALI_ASSERT(W.shape()[1] == 3 * H && U.shape()[1] == 3 * H && b.shape()[0] == 3 * H && U.shape()[0] == H && W.shape()[0] == x.shape()[1] &&
                    x.shape()[0] == h.shape()[0],
                "gru_step: inconsistent shapes");
    for (const Array* a : {&x, &h, &W, &U, &b}) a->eval();
    Array px = dot(x, W);                          // [B, 3H]
    Array ph = dot(h, U.slice(1, 0, 2 * H));       // [B, 2H]: reset and update see h itself
    px.eval();
    ph.eval();
    auto bias = [&](int k) { return b.slice(0, k * H, (k + 1) * H).expand_dims(0); };
    auto cols = [&](const Array& a, int k) { return a.slice(1, k * H, (k + 1) * H); };
    Array reset_state = eltmul(sigmoid(add(add(cols(px, 0), cols(ph, 0)), bias(0))), h);
    Array pc = dot(reset_state, U.slice(1, 2 * H, 3 * H));
    pc.eval();
    Array update = sigmoid(add(add(cols(px, 1), cols(ph, 1)), bias(1)));
    Array candidate = tanh(add(add(cols(px, 2), pc), bias(2)));
    Array h_new = add(eltmul(h, subtract(Array(1.0), update)), eltmul(candidate, update));
    h_new.eval();
    return h_new;
}

// GRU::activate_sequence (dali/layers/gru.cpp:59-64): the step applied to every x(t) in turn, the state carried along.
// What does not depend on the state, x(t).W for all three layers, is one product over the whole sequence; a step is
// then the recurrent products and the two gate kernels of gru_step.
GRUSequence gru_sequence(const Array& xs, const Array& h0, const Array& W, const Array& U, const Array& b) {
    DALI_ASSERT(xs.ndim() == 3 && h0.ndim() == 2 && W.ndim() == 2 && U.ndim() == 2 && b.ndim() == 1,
                "gru_sequence: xs must be [T, B, I], h0 a matrix, W and U matrices, b a vector");
    const int T = xs.shape()[0], Bn = xs.shape()[1], In = xs.shape()[2], H = h0.shape()[1];
    DALI_ASSERT(T >= 1 && h0.shape()[0] == Bn && W.shape()[0] == In && W.shape()[1] == 3 * H && U.shape()[0] == H && U.shape()[1] == 3 * H &&
                    b.shape()[0] == 3 * H,
                "gru_sequence: inconsistent shapes");
    for (const Array* a : {&xs, &h0, &W, &U, &b}) a->eval();
    // Small batches: the recurrent half of the whole sequence as one persistent launch (weights in the registers of the compute
    // units, two grid barriers per step), the input half with the bias as one product in front of it.
    {
        auto dense = [](const Array& a) { return a.is_buffer() && a.contiguous_memory() && a.dtype() == DTYPE_FLOAT; };
        const char* persistent_env = getenv("DALI_HIP_GRU_PERSISTENT");  // read per call: a benchmark times both forms in one process
        const bool persistent_off = persistent_env != nullptr && std::string(persistent_env) == "0";
        Array seq = xs.is_buffer() && xs.contiguous_memory() ? xs : xs.ascontiguousarray();
        if (!persistent_off && !dry_run() && T >= 2 && dense(seq) && dense(h0) && dense(W) && dense(U) && dense(b) && h0.offset() % 4 == 0 &&
            ((int64_t)Bn * H) % 4 == 0 && dali_hip_gru_recurrent_persistent_supported(Bn, H) == 2) {
            Array pre = add(dot(seq.reshape({T * Bn, In}), W), b.expand_dims(0));
            pre.eval();
            Array states({T, Bn, H}, DTYPE_FLOAT), scratch({T, Bn, H}, DTYPE_FLOAT);
            gru_recurrent_persistent(pre.reshape({T, Bn, 3 * H}), U, h0, states, scratch);
            GRUSequence out;
            out.states = states;
            out.last = states[T - 1];
            return out;
        }
    }
    Array px_all = dot(xs.reshape({T * Bn, In}), W);  // [T B, 3H]
    px_all.eval();
    auto bias = [&](int k) { return b.slice(0, k * H, (k + 1) * H).expand_dims(0); };
    auto cols = [&](const Array& a, int k) { return a.slice(1, k * H, (k + 1) * H); };
    Array states = Array({T, Bn, H}, DTYPE_FLOAT);
    Array h = h0;
    for (int t = 0; t < T; ++t) {
        Array px = px_all.slice(0, t * Bn, (t + 1) * Bn);
        Array ph = dot(h, U.slice(1, 0, 2 * H));
        ph.eval();
        Array reset_state = eltmul(sigmoid(add(add(cols(px, 0), cols(ph, 0)), bias(0))), h);
        Array pc = dot(reset_state, U.slice(1, 2 * H, 3 * H));
        pc.eval();
        Array update = sigmoid(add(add(cols(px, 1), cols(ph, 1)), bias(1)));
        Array candidate = tanh(add(add(cols(px, 2), pc), bias(2)));
        Array h_t = states.pluck_axis(0, t);
        h_t.assign(add(eltmul(h, subtract(Array(1.0), update)), eltmul(candidate, update)));
        h_t.eval();
        h = h_t;
    }
    GRUSequence out;
    out.states = states;
    out.last = h;
    return out;
}

}  // namespace op
}  // namespace dali
