// Host-side mirror of Weed's tensor / op / module interface over the HIP device library (see weed.hpp).
#include "weed.hpp"

#include "weed_hip.h"

#include <algorithm>
#include <limits>
#include <cmath>
#include <random>

namespace Weed {

// ---------------------------------------------------------------------------------------------------------
// device
// ---------------------------------------------------------------------------------------------------------

HipDevice::HipDevice()
    : device_id(0)
{
    check(weed_hip_init(0));
    char buf[256] = { 0 };
    if (weed_hip_device_name(buf, sizeof(buf)) == WEED_HIP_OK) {
        name = buf;
    }
}

HipDevice &HipDevice::Instance()
{
    static HipDevice dev;
    return dev;
}

void HipDevice::check(int status)
{
    if (status == WEED_HIP_OK) {
        return;
    }
    const std::string msg = weed_hip_last_error();
    switch (status) {
    case WEED_HIP_EINVAL:
        throw std::invalid_argument(msg);
    case WEED_HIP_ENOMEM:
        throw bad_alloc(msg);
    case WEED_HIP_ECAPACITY:
        throw std::out_of_range(msg);
    default:
        throw std::runtime_error(msg);
    }
}

void HipDevice::finish()
{
    std::lock_guard<std::recursive_mutex> lock(mutex);
    check(weed_hip_sync());
}

namespace {

typedef std::lock_guard<std::recursive_mutex> DeviceLock;
#define WEED_DEVICE_LOCK() DeviceLock device_lock(HipDevice::Instance().mutex)

DeviceTag resolve(DeviceTag dtag) { return (dtag == CPU) ? CPU : GPU; }

real1 *device_ptr(const Tensor &t, const char *who)
{
    if (!t.storage) {
        throw std::invalid_argument(std::string(who) + ": tensor has no storage");
    }
    if (t.storage->dtype != DType::REAL) {
        throw std::invalid_argument(std::string(who) + ": only real tensors are supported");
    }
    if (t.storage->device != GPU) {
        throw std::domain_error(std::string(who) + ": this build computes on the GPU only; move the tensor with cast(GPU)");
    }
    return static_cast<GpuRealStorage *>(t.storage.get())->buffer;
}

void validate_all_same_device(std::initializer_list<const Tensor *> ts, const char *who)
{
    DeviceTag d = NONE_DEVICE;
    for (const Tensor *t : ts) {
        if (!t->storage) {
            throw std::invalid_argument(std::string(who) + ": tensor has no storage");
        }
        if (d == NONE_DEVICE) {
            d = t->storage->device;
        } else if (d != t->storage->device) {
            throw std::invalid_argument(std::string("Tensor device mismatch in ") + who + "!");
        }
    }
}

symint wrap_axis(symint axis, size_t rank, const char *who)
{
    if (axis < 0) {
        axis += (symint)rank;
    }
    if (axis < 0 || (size_t)axis >= rank) {
        throw std::invalid_argument(std::string(who) + ": axis out of range");
    }
    return axis;
}

TensorPtr allocate(const std::vector<tcapint> &shape, const Tensor &like)
{
    return std::make_shared<Tensor>(shape, Tensor::full_contiguous_stride(shape), false, false, DType::REAL,
        like.storage->device, like.storage->get_device_id());
}

// A tensor whose LAST dimension is the contiguous one (the reversed view of a column-major allocation): for
// intermediates that only device kernels see.
TensorPtr allocate_last_fastest(const std::vector<tcapint> &shape, const Tensor &like)
{
    TensorPtr t = allocate(std::vector<tcapint>(shape.rbegin(), shape.rend()), like);
    std::reverse(t->shape.begin(), t->shape.end());
    std::reverse(t->stride.begin(), t->stride.end());
    return t;
}

void elementwise(int op, const Tensor &a, const Tensor *b, Tensor &out, const char *who)
{
    // operands are right-aligned against out's shape; a dimension of size 1 repeats (stride 0)
    const size_t rank = out.shape.size();
    if (rank > 8U) {
        throw std::invalid_argument(std::string(who) + ": rank above 8");
    }
    auto aligned = [&](const Tensor &t, std::vector<uint32_t> &str) {
        if (t.shape.size() > rank) {
            throw std::invalid_argument(std::string(who) + ": operand rank exceeds output rank");
        }
        const size_t pad = rank - t.shape.size();
        str.assign(rank, 0U);
        for (size_t i = 0; i < t.shape.size(); ++i) {
            if (t.shape[i] == out.shape[pad + i]) {
                str[pad + i] = (t.shape[i] == 1U) ? 0U : t.stride[i];
            } else if (t.shape[i] != 1U) {
                throw std::invalid_argument(std::string(who) + ": shapes cannot be broadcast together");
            }
        }
    };
    std::vector<uint32_t> as, bs, os(rank);
    aligned(a, as);
    if (b) {
        aligned(*b, bs);
    }
    for (size_t i = 0; i < rank; ++i) {
        os[i] = (out.shape[i] == 1U) ? 0U : out.stride[i];
    }
    real1 *ap = device_ptr(a, who), *op_ = device_ptr(out, who);
    real1 *bp = b ? device_ptr(*b, who) : nullptr;
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_elementwise_f32(op, (uint32_t)rank, out.shape.data(), ap, a.offset, as.data(), bp,
        b ? b->offset : 0U, b ? bs.data() : nullptr, op_, out.offset, os.data()));
}

std::vector<tcapint> broadcast_shape(const Tensor &a, const Tensor &b, const char *who)
{
    const size_t rank = std::max(a.shape.size(), b.shape.size());
    std::vector<tcapint> shp(rank, 1U);
    for (const Tensor *t : { &a, &b }) {
        const size_t pad = rank - t->shape.size();
        for (size_t i = 0; i < t->shape.size(); ++i) {
            tcapint &o = shp[pad + i];
            if (o == 1U) {
                o = t->shape[i];
            } else if (t->shape[i] != 1U && t->shape[i] != o) {
                throw std::invalid_argument(std::string(who) + ": shapes cannot be broadcast together");
            }
        }
    }
    return shp;
}

TensorPtr binary(int op, const TensorPtr &a, const TensorPtr &b, const char *who)
{
    validate_all_same_device({ a.get(), b.get() }, who);
    TensorPtr out = allocate(broadcast_shape(*a, *b, who), *a);
    elementwise(op, *a, b.get(), *out, who);
    return out;
}

} // namespace

// ---------------------------------------------------------------------------------------------------------
// storage
// ---------------------------------------------------------------------------------------------------------

Storage::Storage(StorageType stp, DeviceTag dtg, DType dtp, tcapint n)
    : stype(stp)
    , device(dtg)
    , dtype(dtp)
    , size(n)
{
    if (!size) {
        throw std::invalid_argument("Storage must have size of at least 1!");
    }
}

CpuRealStorage::CpuRealStorage(tcapint n)
    : RealStorage(REAL_CPU_DENSE, CPU, DType::REAL, n)
    , data(n)
{
}

CpuRealStorage::CpuRealStorage(const std::vector<real1> &val)
    : RealStorage(REAL_CPU_DENSE, CPU, DType::REAL, (tcapint)val.size())
    , data(val)
{
}

real1 CpuRealStorage::operator[](const tcapint &idx) const
{
    if (idx >= size) {
        throw std::invalid_argument("CpuStorage::operator[] argument out-of-bounds!");
    }
    return data[idx];
}

void CpuRealStorage::write(const tcapint &idx, const real1 &val)
{
    if (idx >= size) {
        throw std::invalid_argument("CpuStorage::write argument out-of-bounds!");
    }
    data[idx] = val;
}

void CpuRealStorage::add(const tcapint &idx, const real1 &val) { write(idx, (*this)[idx] + val); }
void CpuRealStorage::FillZeros() { std::fill(data.begin(), data.end(), ZERO_R1); }
void CpuRealStorage::FillOnes() { std::fill(data.begin(), data.end(), ONE_R1); }
void CpuRealStorage::FillValue(const real1 &v) { std::fill(data.begin(), data.end(), v); }
StoragePtr CpuRealStorage::gpu(int64_t did) { return std::make_shared<GpuRealStorage>(data, did); }

GpuRealStorage::GpuRealStorage(tcapint n, int64_t did_)
    : RealStorage(REAL_GPU_DENSE, GPU, DType::REAL, n)
    , buffer(nullptr)
    , did(did_ < 0 ? HipDevice::Instance().device_id : did_)
{
    WEED_DEVICE_LOCK();
    void *p = nullptr;
    HipDevice::check(weed_hip_malloc(&p, sizeof(real1) * (size_t)n));
    buffer = static_cast<real1 *>(p);
}

GpuRealStorage::GpuRealStorage(const std::vector<real1> &val, int64_t did_)
    : GpuRealStorage((tcapint)val.size(), did_)
{
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_h2d(buffer, val.data(), sizeof(real1) * val.size()));
}

GpuRealStorage::~GpuRealStorage()
{
    if (buffer) {
        WEED_DEVICE_LOCK();
        (void)weed_hip_free(buffer);
    }
}

real1 GpuRealStorage::operator[](const tcapint &idx) const
{
    if (idx >= size) {
        throw std::invalid_argument("GpuStorage::operator[] argument out-of-bounds!");
    }
    WEED_DEVICE_LOCK();
    real1 v = ZERO_R1;
    HipDevice::check(weed_hip_memcpy_d2h(&v, buffer + idx, sizeof(real1)));
    return v;
}

void GpuRealStorage::write(const tcapint &idx, const real1 &val)
{
    if (idx >= size) {
        throw std::invalid_argument("GpuStorage::write argument out-of-bounds!");
    }
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_h2d(buffer + idx, &val, sizeof(real1)));
}

void GpuRealStorage::add(const tcapint &idx, const real1 &val) { write(idx, (*this)[idx] + val); }

void GpuRealStorage::FillZeros()
{
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memset(buffer, 0, sizeof(real1) * (size_t)size));
}

void GpuRealStorage::FillValue(const real1 &v)
{
    const std::vector<real1> host(size, v);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_h2d(buffer, host.data(), sizeof(real1) * host.size()));
}

void GpuRealStorage::FillOnes() { FillValue(ONE_R1); }

StoragePtr GpuRealStorage::cpu()
{
    std::shared_ptr<CpuRealStorage> host = std::make_shared<CpuRealStorage>(size);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_d2h(host->data.data(), buffer, sizeof(real1) * (size_t)size));
    return host;
}

CpuIntStorage::CpuIntStorage(tcapint n)
    : IntStorage(INT_CPU_DENSE, CPU, DType::INT, n)
    , data(n)
{
}

CpuIntStorage::CpuIntStorage(const std::vector<symint> &val)
    : IntStorage(INT_CPU_DENSE, CPU, DType::INT, (tcapint)val.size())
    , data(val)
{
}

symint CpuIntStorage::operator[](const tcapint &idx) const
{
    if (idx >= size) {
        throw std::invalid_argument("CpuStorage::operator[] argument out-of-bounds!");
    }
    return data[idx];
}

void CpuIntStorage::write(const tcapint &idx, const symint &val)
{
    if (idx >= size) {
        throw std::invalid_argument("CpuStorage::write argument out-of-bounds!");
    }
    data[idx] = val;
}

void CpuIntStorage::add(const tcapint &idx, const symint &val) { write(idx, (*this)[idx] + val); }
void CpuIntStorage::FillZeros() { std::fill(data.begin(), data.end(), 0); }
void CpuIntStorage::FillOnes() { std::fill(data.begin(), data.end(), 1); }
void CpuIntStorage::FillValue(const symint &v) { std::fill(data.begin(), data.end(), v); }
StoragePtr CpuIntStorage::gpu(int64_t did) { return std::make_shared<GpuIntStorage>(data, did); }

GpuIntStorage::GpuIntStorage(tcapint n, int64_t did_)
    : IntStorage(INT_GPU_DENSE, GPU, DType::INT, n)
    , buffer(nullptr)
    , did(did_ < 0 ? HipDevice::Instance().device_id : did_)
{
    WEED_DEVICE_LOCK();
    void *p = nullptr;
    HipDevice::check(weed_hip_malloc(&p, sizeof(symint) * (size_t)n));
    buffer = static_cast<symint *>(p);
}

GpuIntStorage::GpuIntStorage(const std::vector<symint> &val, int64_t did_)
    : GpuIntStorage((tcapint)val.size(), did_)
{
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_h2d(buffer, val.data(), sizeof(symint) * val.size()));
}

GpuIntStorage::~GpuIntStorage()
{
    if (buffer) {
        WEED_DEVICE_LOCK();
        (void)weed_hip_free(buffer);
    }
}

symint GpuIntStorage::operator[](const tcapint &idx) const
{
    if (idx >= size) {
        throw std::invalid_argument("GpuStorage::operator[] argument out-of-bounds!");
    }
    WEED_DEVICE_LOCK();
    symint v = 0;
    HipDevice::check(weed_hip_memcpy_d2h(&v, buffer + idx, sizeof(symint)));
    return v;
}

void GpuIntStorage::write(const tcapint &, const symint &) { throw std::domain_error("Don't use GPU-based Storage::write()!"); }
void GpuIntStorage::add(const tcapint &, const symint &) { throw std::domain_error("Don't use GPU-based Storage::add()!"); }

void GpuIntStorage::FillZeros()
{
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memset(buffer, 0, sizeof(symint) * (size_t)size));
}

void GpuIntStorage::FillValue(const symint &v)
{
    const std::vector<symint> host(size, v);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_h2d(buffer, host.data(), sizeof(symint) * host.size()));
}

void GpuIntStorage::FillOnes() { FillValue(1); }

StoragePtr GpuIntStorage::cpu()
{
    std::shared_ptr<CpuIntStorage> host = std::make_shared<CpuIntStorage>(size);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_memcpy_d2h(host->data.data(), buffer, sizeof(symint) * (size_t)size));
    return host;
}

// ---------------------------------------------------------------------------------------------------------
// tensor
// ---------------------------------------------------------------------------------------------------------

bool Tensor::is_contiguous(const std::vector<tcapint> &shp, const std::vector<tcapint> &s)
{
    tcapint st = 1U;
    for (size_t i = 0U; i < s.size(); ++i) {
        if (shp[i] == 1U) {
            continue; // any stride addresses the single element
        }
        if (s[i] != st) {
            return false;
        }
        st *= shp[i];
    }
    return true;
}

// Number of elements of a shape, computed in 64 bits.  Sizes, strides and offsets are tcapint (32 bits, as in the
// reference's default build, include/common/weed_types.hpp:48-66): a shape whose element count does not fit would
// wrap silently and under-allocate, so it is refused here, before any storage exists or any kernel runs.
uint64_t Tensor::checked_elements(const std::vector<tcapint> &shp)
{
    uint64_t n = 1U;
    for (const tcapint &s : shp) {
        n *= (uint64_t)s;
        if (n > (uint64_t)std::numeric_limits<tcapint>::max()) {
            throw std::invalid_argument("Tensor: shape has more elements than a 32-bit index can address");
        }
    }
    return n;
}

std::vector<tcapint> Tensor::full_contiguous_stride(const std::vector<tcapint> &shp)
{
    (void)checked_elements(shp);
    std::vector<tcapint> str(shp.size());
    tcapint run = 1U;
    for (size_t i = 0U; i < shp.size(); ++i) {
        str[i] = (shp[i] == 1U) ? 0U : run;
        run *= shp[i];
    }
    return str;
}

Tensor::Tensor(const std::vector<tcapint> &shp, const std::vector<tcapint> &str, const bool &rg, const bool &,
    const DType &dtype, const DeviceTag &dtag, const int64_t &did)
    : shape(shp)
    , stride(str)
    , requires_grad(rg)
{
    if (shape.size() != stride.size()) {
        throw std::invalid_argument("Tensor shape vector must have same length as stride vector!");
    }
    if (dtype != DType::REAL) {
        throw std::invalid_argument("Tensor: only real tensors are supported");
    }
    if (!is_contiguous(shp, str)) {
        throw std::invalid_argument("Initial tensor shape and stride must be contiguous!");
    }
    const tcapint n = get_size();
    if (resolve(dtag) == GPU) {
        storage = std::make_shared<GpuRealStorage>(n, did);
    } else {
        storage = std::make_shared<CpuRealStorage>(n);
    }
}

Tensor::Tensor(const std::vector<real1> &val, const std::vector<tcapint> &shp, const bool &rg, const DeviceTag &dtag,
    const int64_t &did)
    : shape(shp)
    , stride(full_contiguous_stride(shp))
    , requires_grad(rg)
{
    if (get_size() != val.size()) {
        throw std::invalid_argument("Tensor value vector must match the size implied by its shape!");
    }
    if (resolve(dtag) == GPU) {
        storage = std::make_shared<GpuRealStorage>(val, did);
    } else {
        storage = std::make_shared<CpuRealStorage>(val);
    }
}

Tensor::Tensor(const real1 &val, const bool &rg, const DeviceTag &dtag, const int64_t &did)
    : Tensor(std::vector<real1>{ val }, std::vector<tcapint>{ 1U }, rg, dtag, did)
{
}

tcapint Tensor::get_size() const
{
    return shape.empty() ? 0U : (tcapint)checked_elements(shape);
}

bool Tensor::is_scalar() const { return get_size() == 1U; }

tcapint Tensor::get_storage_index(const tcapint &idx) const
{
    tcapint curr = idx;
    tcapint stor = offset;
    for (size_t i = 0U; (i < shape.size()) && curr; ++i) {
        stor += (curr % shape[i]) * stride[i];
        curr /= shape[i];
    }
    if (curr) {
        throw std::invalid_argument("Tensor index out-of-range!");
    }
    return stor;
}

real1 Tensor::get_item() const
{
    if (!is_scalar()) {
        throw std::invalid_argument("Tensor::get_item(): not a one-element tensor");
    }
    return (*static_cast<RealStorage *>(storage.get()))[offset];
}

TensorPtr Tensor::operator[](const tcapint &idx) const
{
    if (idx >= shape.back()) {
        throw std::invalid_argument("Tensor index out-of-range!");
    }
    TensorPtr v = std::make_shared<Tensor>(*this);
    v->offset += idx * stride.back();
    v->shape.pop_back();
    v->stride.pop_back();
    if (v->shape.empty()) {
        v->shape = { 1U };
        v->stride = { 0U };
    }
    return v;
}

std::vector<real1> Tensor::to_vector() const
{
    StoragePtr host = storage->cpu();
    const RealStorage &rs = *static_cast<RealStorage *>(host.get());
    const tcapint n = get_size();
    std::vector<real1> out(n);
    for (tcapint i = 0U; i < n; ++i) {
        out[i] = rs[get_storage_index(i)];
    }
    return out;
}

TensorPtr Tensor::cast(const DeviceTag &dtag) const
{
    TensorPtr t = std::make_shared<Tensor>(*this);
    t->storage = (resolve(dtag) == GPU) ? storage->gpu() : storage->cpu();
    return t;
}

TensorPtr Tensor::zeros(const std::vector<tcapint> &shape, const bool &rg, const bool &s, const DType &dtype,
    const DeviceTag &dtag, const int64_t &did)
{
    TensorPtr z = std::make_shared<Tensor>(shape, full_contiguous_stride(shape), rg, s, dtype, dtag, did);
    z->storage->FillZeros();
    return z;
}

TensorPtr Tensor::contiguous(const TensorPtr a)
{
    if (a->is_contiguous()) {
        return a;
    }
    TensorPtr out = allocate(a->shape, *a);
    elementwise(WEED_HIP_EW_COPY, *a, nullptr, *out, "Tensor::contiguous");
    return out;
}

TensorPtr Tensor::compact(const TensorPtr a)
{
    if (a->is_contiguous() && a->offset == 0U && a->storage->size == a->get_size()) {
        return a;
    }
    TensorPtr out = allocate(a->shape, *a);
    elementwise(WEED_HIP_EW_COPY, *a, nullptr, *out, "Tensor::compact");
    return out;
}

TensorPtr Tensor::reshape(const TensorPtr a, const std::vector<symint> &s)
{
    TensorPtr out = a->is_contiguous() ? std::make_shared<Tensor>(*a) : contiguous(a);
    const tcapint total = out->get_size();
    std::vector<tcapint> shp(s.size());
    symint infer = -1;
    uint64_t known = 1U;
    for (size_t i = 0U; i < s.size(); ++i) {
        if (s[i] < 0) {
            if (infer >= 0) {
                throw std::invalid_argument("Tensor::reshape(): only one -1 dimension allowed");
            }
            infer = (symint)i;
        } else {
            shp[i] = (tcapint)s[i];
            known *= (uint64_t)(tcapint)s[i];
            if (known > (uint64_t)std::numeric_limits<tcapint>::max()) {
                throw std::invalid_argument("Tensor::reshape(): sizes do not match");
            }
        }
    }
    if (infer >= 0) {
        if (!known || (total % known)) {
            throw std::invalid_argument("Tensor::reshape(): cannot infer dimension size");
        }
        shp[(size_t)infer] = (tcapint)(total / known);
        known *= shp[(size_t)infer];
    }
    if (known != total || shp.empty()) {
        throw std::invalid_argument("Tensor::reshape(): sizes do not match");
    }
    out->shape = shp;
    out->stride = full_contiguous_stride(shp);
    return out;
}

TensorPtr Tensor::transpose(const TensorPtr a)
{
    if (a->shape.size() != 2U) {
        throw std::invalid_argument("Tensor::transpose is only for 2D tensors (and vectors and covectors)!");
    }
    return transpose(a, 0, 1);
}

TensorPtr Tensor::transpose(const TensorPtr a, symint i, symint j)
{
    i = wrap_axis(i, a->shape.size(), "Tensor::transpose");
    j = wrap_axis(j, a->shape.size(), "Tensor::transpose");
    TensorPtr out = std::make_shared<Tensor>(*a);
    std::swap(out->shape[(size_t)i], out->shape[(size_t)j]);
    std::swap(out->stride[(size_t)i], out->stride[(size_t)j]);
    return out;
}

TensorPtr Tensor::slice(TensorPtr a, const int64_t &row)
{
    // fixes an index of dimension 0 and drops that dimension
    if (row < 0 || (tcapint)row >= a->shape[0U]) {
        throw std::invalid_argument("Tensor::slice(): row out of range");
    }
    TensorPtr out = std::make_shared<Tensor>(*a);
    out->offset += (tcapint)row * a->stride[0U];
    out->shape.erase(out->shape.begin());
    out->stride.erase(out->stride.begin());
    if (out->shape.empty()) {
        out->shape = { 1U };
        out->stride = { 0U };
    }
    return out;
}

TensorPtr Tensor::slice(TensorPtr a, int64_t axis, const tcapint &start, const tcapint &length)
{
    const size_t ax = (size_t)wrap_axis((symint)axis, a->shape.size(), "Tensor::slice");
    if (!length || (start + length) > a->shape[ax]) {
        throw std::invalid_argument("Tensor::slice(): range out of bounds");
    }
    TensorPtr out = std::make_shared<Tensor>(*a);
    out->offset += start * a->stride[ax];
    out->shape[ax] = length;
    return out;
}

TensorPtr Tensor::softmax(const TensorPtr x, symint axis)
{
    axis = wrap_axis(axis, x->shape.size(), "Tensor::softmax");
    TensorPtr out = allocate(x->shape, *x);
    Weed::softmax((tcapint)axis, *x, *out);
    return out;
}

namespace {
TensorPtr axis_reduce(TensorPtr a, symint axis, void (*op)(const tcapint &, const Tensor &, Tensor &), const char *who)
{
    axis = wrap_axis(axis, a->shape.size(), who);
    std::vector<tcapint> shp = a->shape;
    shp.erase(shp.begin() + axis);
    if (shp.empty()) {
        shp = { 1U };
    }
    TensorPtr out = allocate(shp, *a);
    op((tcapint)axis, *a, *out);
    return out;
}
} // namespace

TensorPtr Tensor::sum(TensorPtr a, symint axis) { return axis_reduce(a, axis, Weed::reduce, "Tensor::sum"); }
TensorPtr Tensor::max(TensorPtr a, symint axis) { return axis_reduce(a, axis, Weed::max, "Tensor::max"); }
TensorPtr Tensor::min(TensorPtr a, symint axis) { return axis_reduce(a, axis, Weed::min, "Tensor::min"); }
TensorPtr Tensor::add(TensorPtr a, TensorPtr b) { return binary(WEED_HIP_EW_ADD, a, b, "Tensor::add"); }
TensorPtr Tensor::sub(TensorPtr a, TensorPtr b) { return binary(WEED_HIP_EW_SUB, a, b, "Tensor::sub"); }
TensorPtr Tensor::mul(TensorPtr a, TensorPtr b) { return binary(WEED_HIP_EW_MUL, a, b, "Tensor::mul"); }
TensorPtr Tensor::div(TensorPtr a, TensorPtr b) { return binary(WEED_HIP_EW_DIV, a, b, "Tensor::div"); }

TensorPtr Tensor::mean(TensorPtr a, symint axis)
{
    axis = wrap_axis(axis, a->shape.size(), "Tensor::mean");
    TensorPtr tmp = sum(a, axis) / (real1)(a->shape[(size_t)axis]);
    // the axis comes back with extent 1 (tensor.cpp:689-691)
    std::vector<symint> shp(a->shape.begin(), a->shape.end());
    shp[(size_t)axis] = 1;
    return reshape(tmp, shp);
}

namespace {
TensorPtr unary(void (*op)(const Tensor &, Tensor &), const TensorPtr &a)
{
    TensorPtr out = allocate(a->shape, *a);
    op(*a, *out);
    return out;
}
void unary_op(int op, const Tensor &a, Tensor &out, const char *who)
{
    validate_all_same_device({ &a, &out }, who);
    if (a.get_size() != out.get_size()) {
        throw std::invalid_argument(std::string("In Weed::") + who + "(a, out), out size does not match input size!");
    }
    elementwise(op, a, nullptr, out, who);
}
} // namespace

TensorPtr Tensor::relu(TensorPtr a) { return unary(Weed::relu, a); }
TensorPtr Tensor::sigmoid(TensorPtr a) { return unary(Weed::sigmoid, a); }
TensorPtr Tensor::tanh(TensorPtr a) { return unary(Weed::tanh, a); }
TensorPtr Tensor::gelu(const TensorPtr x)
{
    // the reference's chain x3 = x * x * x; inner = k2 * (x + k1 * x3); k0 * x * (1 + tanh(inner))
    // (tensor.cpp:841-851) as one kernel that rounds after every operation as the chain does
    TensorPtr out = allocate(x->shape, *x);
    unary_op(WEED_HIP_EW_GELU, *x, *out, "gelu");
    return out;
}

TensorPtr Tensor::matmul(TensorPtr a, TensorPtr b)
{
    if (a->shape.size() < 2U) {
        throw std::invalid_argument("Tensor::matmul requires a to have rank >= 2");
    }
    const size_t rank = a->shape.size();
    if (rank > 2U && b->shape.size() > 2U) {
        // one 2-D product per index of the leading (batch) dimensions (src/tensors/tensor.cpp:1213-1272)
        if (rank != b->shape.size()) {
            throw std::invalid_argument("batched matmul rank mismatch");
        }
        tcapint batch = 1U;
        for (size_t i = 0; i < rank - 2U; ++i) {
            if (a->shape[i] != b->shape[i]) {
                throw std::invalid_argument("batched matmul batch mismatch");
            }
            batch *= a->shape[i];
        }
        const tcapint M = a->shape[rank - 2U], K = a->shape[rank - 1U], N = b->shape[rank - 1U];
        if (K != b->shape[rank - 2U]) {
            throw std::invalid_argument("batched matmul inner dim mismatch");
        }
        std::vector<tcapint> shp(a->shape.begin(), a->shape.end() - 2);
        shp.push_back(M);
        shp.push_back(N);
        TensorPtr out = allocate(shp, *a);
        // The reference calls the 2-D product once per index of the leading dimensions; here the two innermost
        // leading dimensions go to the device as ONE batched launch and only what lies beyond them is looped over.
        validate_all_same_device({ a.get(), b.get(), out.get() }, "MatMulKernel::matmul");
        real1 *ap = device_ptr(*a, "matmul"), *bp = device_ptr(*b, "matmul"), *op = device_ptr(*out, "matmul");
        const size_t lead = rank - 2U;          // leading dimensions
        const size_t inner = lead >= 2U ? 2U : lead; // handled by the device: dimensions [0, inner)
        tcapint nb[2] = { 1U, 1U }, abs_[2] = { 0U, 0U }, bbs[2] = { 0U, 0U }, obs[2] = { 0U, 0U };
        for (size_t dd = 0; dd < inner; ++dd) {
            nb[dd] = a->shape[dd];
            abs_[dd] = a->stride[dd];
            bbs[dd] = b->stride[dd];
            obs[dd] = out->stride[dd];
        }
        tcapint outer = 1U;
        for (size_t dd = inner; dd < lead; ++dd) {
            outer *= a->shape[dd];
        }
        (void)batch;
        WEED_DEVICE_LOCK();
        for (tcapint i = 0U; i < outer; ++i) {
            tcapint aoff = a->offset, boff = b->offset, ooff = out->offset, rem = i;
            for (size_t dd = inner; dd < lead; ++dd) {
                const tcapint c = rem % a->shape[dd];
                rem /= a->shape[dd];
                aoff += c * a->stride[dd];
                boff += c * b->stride[dd];
                ooff += c * out->stride[dd];
            }
            // at most 65535 products per launch: split the second batch dimension if need be
            const tcapint per = nb[0] ? std::max<tcapint>(1U, std::min<tcapint>(nb[1], 65535U / std::max<tcapint>(nb[0], 1U))) : 1U;
            if (nb[0] > 65535U) {
                throw std::invalid_argument("batched matmul: more than 65535 products along one dimension");
            }
            for (tcapint c1 = 0U; c1 < nb[1]; c1 += per) {
                const tcapint n1 = std::min<tcapint>(per, nb[1] - c1);
                const tcapint bshape[2] = { nb[0], n1 };
                HipDevice::check(weed_hip_matmul_batched_f32(bshape, M, N, K, ap, aoff + c1 * abs_[1], a->stride[rank - 2U],
                    a->stride[rank - 1U], abs_, bp, boff + c1 * bbs[1], b->stride[rank - 2U], b->stride[rank - 1U], bbs, op,
                    ooff + c1 * obs[1], out->stride[rank - 2U], out->stride[rank - 1U], obs));
            }
        }
        return out;
    }
    if (b->shape.size() != 2U) {
        throw std::invalid_argument("Tensor::matmul requires b to have rank 2 when a is flattened");
    }
    const tcapint K = a->shape.back(), N = b->shape[1U];
    if (b->shape[0U] != K) {
        throw std::invalid_argument("matmul dimension mismatch");
    }
    TensorPtr a2 = (rank > 2U) ? reshape(a, { -1, (symint)K }) : a;
    TensorPtr out = allocate({ a2->shape[0U], N }, *a2);
    Weed::matmul(*a2, *b, *out);
    if (rank > 2U) {
        std::vector<symint> shp(a->shape.begin(), a->shape.end() - 1);
        shp.push_back((symint)N);
        out = reshape(out, shp);
    }
    return out;
}

TensorPtr operator+(TensorPtr left, TensorPtr right) { return Tensor::add(left, right); }
TensorPtr operator-(TensorPtr left, TensorPtr right) { return Tensor::sub(left, right); }
TensorPtr operator*(TensorPtr left, TensorPtr right) { return Tensor::mul(left, right); }
TensorPtr operator/(TensorPtr left, TensorPtr right) { return Tensor::div(left, right); }
TensorPtr operator/(TensorPtr left, real1 right)
{
    // a scalar operand becomes a one-element tensor on the same device (include/tensors/tensor.hpp:622-624)
    return Tensor::div(left, std::make_shared<Tensor>(right, false, left->storage->device, left->storage->get_device_id()));
}
TensorPtr operator*(real1 left, TensorPtr right)
{
    return Tensor::mul(std::make_shared<Tensor>(left, false, right->storage->device, right->storage->get_device_id()), right);
}
TensorPtr operator>>(TensorPtr left, TensorPtr right) { return Tensor::matmul(left, right); }
TensorPtr operator<<(TensorPtr right, TensorPtr left) { return Tensor::matmul(left, right); }

// ---------------------------------------------------------------------------------------------------------
// ops
// ---------------------------------------------------------------------------------------------------------

void matmul(const Tensor &a, const Tensor &b, Tensor &out)
{
    validate_all_same_device({ &a, &b, &out }, "MatMulKernel::matmul");
    if (a.shape.size() != 2U || b.shape.size() != 2U || out.shape.size() != 2U) {
        throw std::invalid_argument("MatMul is only for matrices with 2 indices!");
    }
    const tcapint M = a.shape[0U], K = a.shape[1U], N = b.shape[1U];
    if (K != b.shape[0U] || out.shape[0U] != M || out.shape[1U] != N) {
        throw std::invalid_argument("MatMul operand dimensions aren't compatible!");
    }
    real1 *ap = device_ptr(a, "matmul"), *bp = device_ptr(b, "matmul"), *op = device_ptr(out, "matmul");
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_matmul_f32(M, N, K, ap, a.offset, a.stride[0U], a.stride[1U], bp, b.offset, b.stride[0U],
        b.stride[1U], op, out.offset, out.stride[0U], out.stride[1U]));
}

void softmax(const tcapint &index, const Tensor &a, Tensor &out)
{
    validate_all_same_device({ &a, &out }, "SoftmaxKernel::softmax_forward");
    if (a.shape != out.shape) {
        throw std::invalid_argument("Tensor shape mismatch in softmax_forward!");
    }
    if (index >= a.shape.size()) {
        throw std::invalid_argument("softmax axis out of range");
    }
    real1 *ap = device_ptr(a, "softmax"), *op = device_ptr(out, "softmax");
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_softmax_f32((uint32_t)a.shape.size(), a.shape.data(), index, ap, a.offset, a.stride.data(),
        op, out.offset, out.stride.data()));
}

namespace {
void axis_op(int op, const tcapint &index, const Tensor &a, Tensor &out, const char *who)
{
    validate_all_same_device({ &a, &out }, who);
    if (index >= a.shape.size()) {
        throw std::invalid_argument(std::string(who) + ": axis out of range");
    }
    std::vector<tcapint> want = a.shape;
    want.erase(want.begin() + index);
    if (want.empty()) {
        want = { 1U };
    }
    if (want != out.shape) {
        throw std::invalid_argument(std::string(who) + ": output shape mismatch");
    }
    std::vector<uint32_t> os(out.stride.begin(), out.stride.end());
    if (a.shape.size() == 1U) {
        os = { 0U };
    } else {
        os.insert(os.begin() + index, 0U);
    }
    real1 *ap = device_ptr(a, who), *op_ = device_ptr(out, who);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_reduce_f32(op, (uint32_t)a.shape.size(), a.shape.data(), index, ap, a.offset,
        a.stride.data(), op_, out.offset, os.data()));
}
} // namespace

void reduce(const tcapint &index, const Tensor &a, Tensor &out) { axis_op(WEED_HIP_REDUCE_SUM, index, a, out, "ReduceKernel::reduce"); }
void max(const tcapint &index, const Tensor &a, Tensor &out) { axis_op(WEED_HIP_REDUCE_MAX, index, a, out, "ReduceKernel::max"); }
void min(const tcapint &index, const Tensor &a, Tensor &out) { axis_op(WEED_HIP_REDUCE_MIN, index, a, out, "ReduceKernel::min"); }

void add(const Tensor &a, const Tensor &b, Tensor &out)
{
    validate_all_same_device({ &a, &b, &out }, "CommutingKernel::commuting");
    elementwise(WEED_HIP_EW_ADD, a, &b, out, "add");
}
void mul(const Tensor &a, const Tensor &b, Tensor &out)
{
    validate_all_same_device({ &a, &b, &out }, "CommutingKernel::commuting");
    elementwise(WEED_HIP_EW_MUL, a, &b, out, "mul");
}
void sub(const Tensor &a, const Tensor &b, Tensor &out)
{
    validate_all_same_device({ &a, &b, &out }, "SubKernel::sub");
    elementwise(WEED_HIP_EW_SUB, a, &b, out, "sub");
}
void div(const Tensor &a, const Tensor &b, Tensor &out)
{
    validate_all_same_device({ &a, &b, &out }, "DivKernel::div");
    elementwise(WEED_HIP_EW_DIV, a, &b, out, "div");
}
void add_in_place(Tensor &a, const Tensor &b)
{
    validate_all_same_device({ &a, &b }, "InPlaceKernel::in_place");
    elementwise(WEED_HIP_EW_ADD, a, &b, a, "add_in_place");
}

void relu(const Tensor &a, Tensor &out) { unary_op(WEED_HIP_EW_RELU, a, out, "relu"); }
void sigmoid(const Tensor &a, Tensor &out) { unary_op(WEED_HIP_EW_SIGMOID, a, out, "sigmoid"); }
void tanh(const Tensor &a, Tensor &out) { unary_op(WEED_HIP_EW_TANH, a, out, "tanh"); }

void triu_fill(Tensor &a, const real1 &val, const tcapint diagonal)
{
    if (a.shape.size() != 2U) {
        throw std::invalid_argument("triu_fill: tensor must be 2D [T, T]");
    }
    real1 *ap = device_ptr(a, "triu_fill");
    WEED_DEVICE_LOCK();
    HipDevice::check(
        weed_hip_triu_fill_f32(a.shape[0U], a.shape[1U], val, diagonal, ap, a.offset, a.stride[0U], a.stride[1U]));
}

// ---------------------------------------------------------------------------------------------------------
// Linear
// ---------------------------------------------------------------------------------------------------------

Linear::Linear(tcapint in_f, tcapint out_f, bool use_bias, bool init_rand, DType dtype, DeviceTag device, int64_t device_id)
    : Module(LINEAR_T)
    , in_features(in_f)
    , out_features(out_f)
{
    if (dtype != DType::REAL) {
        throw std::invalid_argument("Linear: only real parameters are supported");
    }
    std::vector<real1> w((size_t)in_f * out_f, ZERO_R1);
    if (init_rand) {
        // uniform in +-1/sqrt(in_features)
        std::mt19937 rng{ std::random_device{}() };
        const real1 lim = ONE_R1 / std::sqrt((real1)in_f);
        std::uniform_real_distribution<real1> dist(-lim, lim);
        for (real1 &v : w) {
            v = dist(rng);
        }
    }
    weight = std::make_shared<Parameter>(w, std::vector<tcapint>{ in_f, out_f }, true, device, device_id);
    if (use_bias) {
        bias = std::make_shared<Parameter>(
            std::vector<real1>(out_f, ZERO_R1), std::vector<tcapint>{ 1U, out_f }, true, device, device_id);
    }
}

TensorPtr Linear::forward(const TensorPtr x)
{
    const bool plain_bias = bias && bias->shape.size() == 2U && bias->shape[0U] == 1U && bias->shape[1U] == out_features;
    if (!plain_bias || x->shape.size() < 2U || weight->shape.size() != 2U) {
        TensorPtr y = x >> weight;
        if (bias) {
            // unlike Tensor::add in the reference (src/tensors/tensor.cpp:1091), broadcasting never reshapes the bias
            // itself, so the sequence length may change between calls
            y = y + bias;
        }
        return y;
    }
    // `x >> weight` then `+ bias` (src/modules/linear.cpp:86-100) as one launch: the product's epilogue adds the bias
    // to the rounded sum, which gives the same bits as the two separate ops
    const size_t rank = x->shape.size();
    const tcapint K = x->shape.back(), N = weight->shape[1U];
    if (weight->shape[0U] != K) {
        throw std::invalid_argument("matmul dimension mismatch");
    }
    TensorPtr a2 = (rank > 2U) ? Tensor::reshape(x, { -1, (symint)K }) : x;
    TensorPtr out = allocate({ a2->shape[0U], N }, *a2);
    validate_all_same_device({ a2.get(), weight.get(), bias.get(), out.get() }, "Linear::forward");
    real1 *ap = device_ptr(*a2, "Linear::forward"), *wp = device_ptr(*weight, "Linear::forward");
    real1 *bp = device_ptr(*bias, "Linear::forward"), *op = device_ptr(*out, "Linear::forward");
    {
        WEED_DEVICE_LOCK();
        HipDevice::check(weed_hip_linear_f32(a2->shape[0U], N, K, ap, a2->offset, a2->stride[0U], a2->stride[1U], wp,
            weight->offset, weight->stride[0U], weight->stride[1U], bp, bias->offset, bias->stride[1U], op, out->offset,
            out->stride[0U], out->stride[1U]));
    }
    if (rank > 2U) {
        std::vector<symint> shp(x->shape.begin(), x->shape.end() - 1);
        shp.push_back((symint)N);
        out = Tensor::reshape(out, shp);
    }
    return out;
}

namespace {
// weights (in, out) with a column per output, k contiguous; biases (1, out)
bool plain_linear(const Linear &l)
{
    const Parameter *w = l.weight.get(), *b = l.bias.get();
    return w && w->shape.size() == 2U && w->shape[0U] == l.in_features && w->shape[1U] == l.out_features &&
        (w->stride[0U] == 1U || l.in_features == 1U) && (w->stride[1U] == l.in_features || l.out_features == 1U) &&
        (!b || (b->shape.size() == 2U && b->shape[0U] == 1U && b->shape[1U] == l.out_features &&
                (b->stride[1U] == 1U || l.out_features == 1U)));
}
bool lie_side_by_side(const std::vector<LinearPtr> &ls)
{
    if (ls.size() < 2U || !ls[0U] || !plain_linear(*ls[0U])) {
        return false;
    }
    const Linear &first = *ls[0U];
    tcapint cols = 0U;
    for (const LinearPtr &l : ls) {
        if (!l || !plain_linear(*l) || l->in_features != first.in_features || !l->bias != !first.bias ||
            l->weight->storage != first.weight->storage ||
            l->weight->offset != first.weight->offset + cols * first.in_features ||
            (l->bias && (l->bias->storage != first.bias->storage || l->bias->offset != first.bias->offset + cols))) {
            return false;
        }
        cols += l->out_features;
    }
    return true;
}
} // namespace

void place_side_by_side(const std::vector<LinearPtr> &ls)
{
    if (ls.size() < 2U) {
        return;
    }
    tcapint cols = 0U;
    for (const LinearPtr &l : ls) {
        if (!l || !l->weight || !plain_linear(*l) || l->in_features != ls[0U]->in_features || !l->bias != !ls[0U]->bias) {
            throw std::invalid_argument("place_side_by_side(): the modules need plain (in, out) weights of the same "
                                        "in_features, and biases all or none");
        }
        cols += l->out_features;
    }
    if (lie_side_by_side(ls)) {
        return;
    }
    const tcapint in = ls[0U]->in_features;
    for (const LinearPtr &l : ls) {
        validate_all_same_device({ ls[0U]->weight.get(), l->weight.get() }, "place_side_by_side");
        if (l->bias) {
            validate_all_same_device({ ls[0U]->weight.get(), l->bias.get() }, "place_side_by_side");
        }
    }
    TensorPtr w = allocate({ in, cols }, *ls[0U]->weight);
    TensorPtr b = ls[0U]->bias ? allocate({ 1U, cols }, *ls[0U]->bias) : nullptr;
    tcapint at = 0U;
    for (const LinearPtr &l : ls) {
        TensorPtr wv = Tensor::slice(w, 1, at, l->out_features);
        elementwise(WEED_HIP_EW_COPY, *l->weight, nullptr, *wv, "place_side_by_side");
        l->weight->storage = wv->storage;
        l->weight->offset = wv->offset;
        l->weight->stride = wv->stride;
        if (b) {
            TensorPtr bv = Tensor::slice(b, 1, at, l->out_features);
            elementwise(WEED_HIP_EW_COPY, *l->bias, nullptr, *bv, "place_side_by_side");
            l->bias->storage = bv->storage;
            l->bias->offset = bv->offset;
            l->bias->stride = bv->stride;
        }
        at += l->out_features;
    }
}

std::vector<TensorPtr> forward_side_by_side(const std::vector<LinearPtr> &ls, const TensorPtr x)
{
    std::vector<TensorPtr> out;
    if (!lie_side_by_side(ls)) {
        for (const LinearPtr &l : ls) {
            out.push_back(l->forward(x));
        }
        return out;
    }
    tcapint cols = 0U;
    for (const LinearPtr &l : ls) {
        cols += l->out_features;
    }
    // one module over all the columns: views of the shared storages
    Linear all;
    all.in_features = ls[0U]->in_features;
    all.out_features = cols;
    all.weight = std::make_shared<Parameter>();
    static_cast<Tensor &>(*all.weight) = static_cast<const Tensor &>(*ls[0U]->weight);
    all.weight->shape = { all.in_features, cols };
    if (ls[0U]->bias) {
        all.bias = std::make_shared<Parameter>();
        static_cast<Tensor &>(*all.bias) = static_cast<const Tensor &>(*ls[0U]->bias);
        all.bias->shape = { 1U, cols };
    }
    TensorPtr y = all.forward(x);
    tcapint at = 0U;
    for (const LinearPtr &l : ls) {
        out.push_back(Tensor::slice(y, -1, at, l->out_features));
        at += l->out_features;
    }
    return out;
}

std::vector<ParameterPtr> Linear::parameters()
{
    std::vector<ParameterPtr> p{ weight };
    if (bias) {
        p.push_back(bias);
    }
    return p;
}

// ---------------------------------------------------------------------------------------------------------
// RoPE
// ---------------------------------------------------------------------------------------------------------

RoPE::RoPE(const tcapint &head_dim_, const tcapint &max_seq_len_, const real1_f &base_, DeviceTag dtag)
    : Module(ROPE_T)
    , head_dim(head_dim_)
    , max_seq_len(max_seq_len_)
    , base(base_)
{
    if (!head_dim || (head_dim & 1U) || !max_seq_len) {
        throw std::invalid_argument("RoPE: head_dim must be even and max_seq_len positive");
    }
    _build_tables(dtag);
}

void RoPE::_build_tables(DeviceTag dtag)
{
    // theta_i = base^(-2i/head_dim); entry (pos, 2i) = (pos, 2i+1) = cos / sin (pos * theta_i); column-major
    const tcapint half = head_dim >> 1U;
    std::vector<real1> cos_data((size_t)max_seq_len * head_dim), sin_data((size_t)max_seq_len * head_dim);
    for (tcapint pos = 0U; pos < max_seq_len; ++pos) {
        for (tcapint i = 0U; i < half; ++i) {
            const real1_f theta = (real1_f)std::pow(base, -2.0f * (real1_f)i / (real1_f)head_dim);
            const real1_f angle = (real1_f)pos * theta;
            const real1 c = (real1)std::cos(angle), sn = (real1)std::sin(angle);
            for (tcapint e = 0U; e < 2U; ++e) {
                cos_data[pos + (size_t)(2U * i + e) * max_seq_len] = c;
                sin_data[pos + (size_t)(2U * i + e) * max_seq_len] = sn;
            }
        }
    }
    cos_table = std::make_shared<Tensor>(cos_data, std::vector<tcapint>{ max_seq_len, head_dim }, false, dtag);
    sin_table = std::make_shared<Tensor>(sin_data, std::vector<tcapint>{ max_seq_len, head_dim }, false, dtag);
}

void RoPE::apply(const Tensor &x, Tensor &out, tcapint pos0)
{
    if (x.shape.size() != 4U || x.shape[3U] != head_dim || out.shape != x.shape) {
        throw std::invalid_argument("RoPE: input and output must be (B, H, T, head_dim)");
    }
    validate_all_same_device({ &x, &out, cos_table.get(), sin_table.get() }, "RoPE::forward");
    if ((uint64_t)pos0 + x.shape[2U] > max_seq_len) {
        throw std::out_of_range("RoPE: positions beyond max_seq_len");
    }
    real1 *xp = device_ptr(x, "RoPE::forward"), *op = device_ptr(out, "RoPE::forward");
    real1 *cp = device_ptr(*cos_table, "RoPE::forward"), *sp = device_ptr(*sin_table, "RoPE::forward");
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_rope_f32(x.shape.data(), xp, x.offset, x.stride.data(), cp + cos_table->offset,
        sp + sin_table->offset, max_seq_len, pos0, op, out.offset, out.stride.data()));
}

TensorPtr RoPE::forward(const TensorPtr x, tcapint pos0)
{
    if (x->shape.size() != 4U) {
        throw std::invalid_argument("RoPE::forward(): input must be (B, H, T, head_dim)");
    }
    TensorPtr out = allocate(x->shape, *x);
    apply(*x, *out, pos0);
    return out;
}

// ---------------------------------------------------------------------------------------------------------
// quantized cache
// ---------------------------------------------------------------------------------------------------------

DeviceKVCache::DeviceKVCache(int mode, tcapint n_seq_, tcapint n_kv_heads_, tcapint head_dim_, tcapint max_tokens_,
    int k_bits, int v_bits, int k_sign, int v_sign)
    : n_seq(n_seq_)
    , n_kv_heads(n_kv_heads_)
    , head_dim(head_dim_)
    , max_tokens(max_tokens_)
{
    weed_hip_kv_config cfg;
    cfg.mode = mode;
    cfg.n_seq = (int32_t)n_seq_;
    cfg.n_kv_heads = (int32_t)n_kv_heads_;
    cfg.head_dim = (int32_t)head_dim_;
    cfg.max_tokens = (int32_t)max_tokens_;
    cfg.k_bits = k_bits;
    cfg.v_bits = v_bits;
    cfg.k_sign = k_sign;
    cfg.v_sign = v_sign;
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_kv_cache_create(&handle, &cfg));
}

DeviceKVCache::~DeviceKVCache()
{
    if (handle) {
        WEED_DEVICE_LOCK();
        (void)weed_hip_kv_cache_destroy(handle);
    }
}

void QuantizedKVCache::allocate(const tcapint max_outer_, const tcapint d_, const int bits_)
{
    // a single (sequence, kv head) pair holding max_outer rows; both halves of the device object get the same rows
    dev = std::make_shared<DeviceKVCache>(WEED_HIP_KV_UNIFORM, 1U, 1U, d_, max_outer_, bits_, bits_, 0, 0);
    which = 0;
    max_outer = max_outer_;
    d = d_;
    bits = bits_;
    outer = 0U;
    packed.clear();
}

void QuantizedKVCache::write_row(const tcapint row, const real1 *vals)
{
    if (!dev) {
        throw std::domain_error("QuantizedKVCache::write_row(): allocate() first");
    }
    if (dev->n_seq != 1U || dev->n_kv_heads != 1U) {
        throw std::domain_error("QuantizedKVCache::write_row(): rows of a module's cache are written by forward()");
    }
    if (row != outer) {
        throw std::domain_error("QuantizedKVCache::write_row(): rows are append-only on the device");
    }
    GpuRealStorage staging(std::vector<real1>(vals, vals + d));
    const uint32_t str[4] = { 0U, 0U, 0U, 1U };
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_kv_cache_set_scales(dev->handle, block_scale, block_scale));
    HipDevice::check(
        weed_hip_kv_encode_append(dev->handle, 0, 1, 1, staging.buffer, 0U, str, staging.buffer, 0U, str, 0));
    HipDevice::check(weed_hip_sync());
    ++outer;
}

void QuantizedKVCache::read_row(const tcapint row, real1 *vals) const
{
    if (!dev) {
        throw std::domain_error("QuantizedKVCache::read_row(): allocate() first");
    }
    const tcapint pair = row / dev->max_tokens, tok = row % dev->max_tokens;
    if (pair >= dev->n_seq * dev->n_kv_heads) {
        throw std::invalid_argument("QuantizedKVCache::read_row(): row out of range");
    }
    // dequantise [1 sequence, all kv heads, 1 token, d] and keep the wanted head
    const tcapint seq = pair / dev->n_kv_heads, head = pair % dev->n_kv_heads;
    GpuRealStorage staging(dev->n_kv_heads * d);
    const uint32_t str[4] = { 0U, d, 0U, 1U };
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_kv_dequant(dev->handle, which, (int32_t)seq, 1, (int32_t)tok, 1, staging.buffer, 0U, str));
    HipDevice::check(weed_hip_memcpy_d2h(vals, staging.buffer + (size_t)head * d, sizeof(real1) * d));
}

void QuantizedKVCache::sync_packed()
{
    if (!dev) {
        throw std::domain_error("QuantizedKVCache::sync_packed(): allocate() first");
    }
    const tcapint vpw = (tcapint)values_per_word(), wpr = (d + vpw - 1U) / vpw;
    std::vector<int32_t> lens(dev->n_seq);
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_kv_cache_seq_lens(dev->handle, lens.data()));
    const tcapint T = (tcapint)*std::max_element(lens.begin(), lens.end());
    packed.assign((size_t)dev->n_seq * dev->n_kv_heads * T * wpr, 0);
    if (!T) {
        return;
    }
    void *words = nullptr;
    HipDevice::check(weed_hip_malloc(&words, packed.size() * sizeof(int32_t)));
    int st = weed_hip_kv_export_weed_words(dev->handle, which, 0, (int32_t)dev->n_seq, 0, (int32_t)T, (int32_t *)words);
    if (st == WEED_HIP_OK) {
        st = weed_hip_memcpy_d2h(packed.data(), words, packed.size() * sizeof(int32_t));
    }
    (void)weed_hip_free(words);
    HipDevice::check(st);
}

// ---------------------------------------------------------------------------------------------------------
// attention
// ---------------------------------------------------------------------------------------------------------

MultiHeadAttention::MultiHeadAttention(tcapint d_model_, tcapint num_heads_, tcapint num_kv_heads_, tcapint head_dim_,
    DeviceTag dtag, RoPEPtr r, real1_f mask_val_, const int64_t did, const bool _use_kv_cache, int kv_quant_bits_,
    bool use_bias)
    : Module(MULTIHEAD_ATTENTION_T)
    , d_model((symint)d_model_)
    , num_heads((symint)num_heads_)
    , num_kv_heads((symint)(num_kv_heads_ ? num_kv_heads_ : num_heads_))
    , head_dim((symint)(!head_dim_ ? d_model_ / num_heads_ : head_dim_))
    , mask_val(mask_val_)
    , use_kv_cache(_use_kv_cache)
    , kv_quant_bits(kv_quant_bits_)
{
    rope = r;
    if (rope && (symint)rope->head_dim != head_dim) {
        throw std::invalid_argument("MultiHeadAttention: RoPE head_dim does not match");
    }
    if (d_model % num_heads) {
        throw std::invalid_argument("d_model must be divisible by num_heads");
    }
    if (num_heads % num_kv_heads) {
        throw std::invalid_argument("num_heads must be divisible by num_kv_heads");
    }
    const tcapint q_dim = (tcapint)(num_heads * head_dim), kv_dim = (tcapint)(num_kv_heads * head_dim);
    W_q = std::make_shared<Linear>(d_model_, q_dim, use_bias, true, DType::REAL, dtag, did);
    W_k = std::make_shared<Linear>(d_model_, kv_dim, use_bias, true, DType::REAL, dtag, did);
    W_v = std::make_shared<Linear>(d_model_, kv_dim, use_bias, true, DType::REAL, dtag, did);
    W_o = std::make_shared<Linear>(q_dim, d_model_, use_bias, true, DType::REAL, dtag, did);
    for (const LinearPtr &l : { W_q, W_k, W_v, W_o }) {
        const std::vector<ParameterPtr> p = l->parameters();
        param_vector.insert(param_vector.end(), p.begin(), p.end());
    }
    if (mask_val == ZERO_R1) {
        mask_val = -1.701411835e38f; // -2^127 (multihead_attention.hpp:109-110 at fp32)
    }
}

MultiHeadAttention::MultiHeadAttention()
    : Module(MULTIHEAD_ATTENTION_T)
    , d_model(0)
    , num_heads(0)
    , num_kv_heads(0)
    , head_dim(0)
    , mask_val(ZERO_R1)
    , use_kv_cache(true)
{
}

MultiHeadAttention::~MultiHeadAttention()
{
    if (lens_dev) {
        WEED_DEVICE_LOCK();
        (void)weed_hip_free(lens_dev);
    }
}

void MultiHeadAttention::reset_cache()
{
    k_cache = nullptr;
    v_cache = nullptr;
    cache_len = 0U;
    max_seq_len = 0U;
    k_rotation.clear();
    v_rotation.clear();
    v_rotation_trans.clear();
    k_rot_dev = nullptr;
    v_rot_dev = nullptr;
    v_rot_t_dev = nullptr;
    k_qcache = QuantizedKVCache{};
    v_qcache = QuantizedKVCache{};
}

void MultiHeadAttention::set_tables(int which, const std::vector<real1> &bounds, const std::vector<real1> &levels,
    const std::vector<real1> &recon)
{
    if (which != 0 && which != 1) {
        throw std::invalid_argument("MultiHeadAttention::set_tables(): which must be 0 (keys) or 1 (values)");
    }
    if (kv_coder != KV_LLOYDMAX) {
        throw std::invalid_argument("MultiHeadAttention::set_tables(): the uniform coder has no tables");
    }
    const int bits = which ? (v_bits ? v_bits : kv_quant_bits) : (k_bits ? k_bits : kv_quant_bits);
    const bool sign = which ? v_sign : k_sign;
    if (bits < 1 || bits > 4 || bounds.size() != (size_t)(1 << bits) - 1U || levels.size() != (size_t)1 << bits
        || recon.size() != (size_t)1 << (bits + (sign ? 1 : 0))) {
        throw std::invalid_argument("MultiHeadAttention::set_tables(): table sizes do not match the code width");
    }
    if (cache_len) {
        throw std::logic_error("MultiHeadAttention::set_tables(): the cache already holds tokens; reset_cache() first");
    }
    custom_tables[which] = CoderTables{ bounds, levels, recon };
    if (k_qcache.dev) {
        WEED_DEVICE_LOCK();
        std::vector<real1> rounded(recon.size());
        HipDevice::check(weed_hip_kv_cache_set_tables(k_qcache.dev->handle, which, bounds.data(), levels.data(), recon.data(),
            rounded.data()));
    }
}

void MultiHeadAttention::fuse_projections() { place_side_by_side({ W_q, W_k, W_v }); }

TensorPtr MultiHeadAttention::forward(const TensorPtr x)
{
    // x: (B, T, d_model)
    if (x->shape.size() != 3U || (symint)x->shape[2U] != d_model) {
        throw std::invalid_argument("MultiHeadAttention::forward(): input must be (B, T, d_model)");
    }
    const symint B = (symint)x->shape[0U], T = (symint)x->shape[1U];

    // (one product when fuse_projections() laid the three weights side by side)
    const std::vector<TensorPtr> qkv = forward_side_by_side({ W_q, W_k, W_v }, x);
    TensorPtr Q = qkv[0U], K = qkv[1U], V = qkv[2U];

    Q = Tensor::reshape(Q, { B, T, num_heads, head_dim });
    K = Tensor::reshape(K, { B, T, num_kv_heads, head_dim });
    V = Tensor::reshape(V, { B, T, num_kv_heads, head_dim });

    if (rope) {
        // optional RoPE on the (B, heads, T, head_dim) views, at the tokens' positions in the sequence
        const tcapint pos0 = use_kv_cache ? cache_len : 0U;
        if (use_kv_cache && !max_seq_len) {
            max_seq_len = rope->max_seq_len; // the reference's default capacity with RoPE (cpp:173)
        }
        // written straight into fresh contiguous (B, T, heads, head_dim) tensors through transposed views
        for (TensorPtr *t : { &Q, &K }) {
            TensorPtr fresh = allocate((*t)->shape, **t);
            TensorPtr fresh_view = Tensor::transpose(fresh, 1, 2);
            rope->apply(*Tensor::transpose(*t, 1, 2), *fresh_view, pos0);
            *t = fresh;
        }
    }

    TensorPtr out = (use_kv_cache && kv_quant_bits > 0) ? forward_quantized(Q, K, V, B, T) : forward_dense(Q, K, V, B, T);

    // (B, T, num_heads * head_dim)
    out = Tensor::reshape(out, { B, T, num_heads * head_dim });
    return W_o->forward(out);
}

// Quantized cache: rotate + encode + append the new tokens, then one fused kernel per query position over the
// packed rows (multihead_attention.cpp:169-277, 291-348 collapse into these calls).  Q, K, V arrive as contiguous
// (B, T, heads, head_dim) tensors; the (B, heads, T, head_dim) views the reference forms by transpose are expressed
// through strides.  Returns (B, T, num_heads, head_dim), contiguous.
TensorPtr MultiHeadAttention::forward_quantized(TensorPtr Q, TensorPtr K, TensorPtr V, symint B, symint T)
{
    const tcapint hd = (tcapint)head_dim, Hkv = (tcapint)num_kv_heads, Hq = (tcapint)num_heads;
    const tcapint uB = (tcapint)B, uT = (tcapint)T;
    device_ptr(*Q, "MultiHeadAttention::forward");
    WEED_DEVICE_LOCK();

    if (!k_qcache.dev) {
        if (!max_seq_len) {
            max_seq_len = 2048U;
        }
        cache_len = 0U;
        const int kb = k_bits ? k_bits : kv_quant_bits, vb = v_bits ? v_bits : kv_quant_bits;
        const bool lloyd = kv_coder == KV_LLOYDMAX;
        DeviceKVCachePtr dev = std::make_shared<DeviceKVCache>(lloyd ? WEED_HIP_KV_LLOYDMAX : WEED_HIP_KV_UNIFORM, uB, Hkv,
            hd, max_seq_len, kb, vb, (lloyd && k_sign) ? 1 : 0, (lloyd && v_sign) ? 1 : 0);
        if (k_rotation.size() == (size_t)hd * hd && v_rotation.size() == (size_t)hd * hd) {
            k_rot_dev = std::make_shared<GpuRealStorage>(k_rotation);
            v_rot_dev = std::make_shared<GpuRealStorage>(v_rotation);
        } else {
            uint32_t seed = rotation_seed ? rotation_seed : (uint32_t)std::random_device{}();
            k_rot_dev = std::make_shared<GpuRealStorage>(hd * hd);
            v_rot_dev = std::make_shared<GpuRealStorage>(hd * hd);
            HipDevice::check(weed_hip_make_rotation(seed, hd, k_rot_dev->buffer));
            HipDevice::check(weed_hip_make_rotation(seed + 0x9e3779b9U, hd, v_rot_dev->buffer));
            k_rotation = static_cast<CpuRealStorage *>(k_rot_dev->cpu().get())->data;
            v_rotation = static_cast<CpuRealStorage *>(v_rot_dev->cpu().get())->data;
        }
        v_rotation_trans.resize((size_t)hd * hd);
        for (tcapint i = 0U; i < hd; ++i) {
            for (tcapint j = 0U; j < hd; ++j) {
                v_rotation_trans[(size_t)i * hd + j] = v_rotation[(size_t)j * hd + i];
            }
        }
        HipDevice::check(weed_hip_kv_cache_set_rotations(dev->handle, k_rot_dev->buffer, v_rot_dev->buffer));
        for (int which = 0; which < 2; ++which) {
            const CoderTables &t = custom_tables[which];
            if (!t.bounds.empty()) {
                std::vector<real1> rounded(t.recon.size());
                HipDevice::check(weed_hip_kv_cache_set_tables(dev->handle, which, t.bounds.data(), t.levels.data(),
                    t.recon.data(), rounded.data()));
            }
        }
        for (QuantizedKVCache *qc : { &k_qcache, &v_qcache }) {
            qc->dev = dev;
            qc->which = (qc == &v_qcache) ? 1 : 0;
            qc->d = hd;
            qc->bits = qc->which ? vb : kb;
            qc->max_outer = uB * Hkv * max_seq_len;
            qc->outer = 0U;
        }
    }
    weed_hip_kv_cache *cache = k_qcache.dev->handle;
    if (k_qcache.dev->n_seq != uB) {
        throw std::invalid_argument("MultiHeadAttention::forward(): batch size changed while the KV cache is live");
    }

    // element (b, h, t, j) of the logical (B, heads, T, head_dim) views
    const uint32_t kv_str[4] = { 1U, uB * uT, uB, uB * uT * Hkv };
    const uint32_t kv_shape[4] = { uB, Hkv, uT, hd };
    real1 *kp = device_ptr(*K, "MultiHeadAttention::forward"), *vp = device_ptr(*V, "MultiHeadAttention::forward");
    if (kv_coder == KV_UNIFORM) {
        // rotate in the reference's rounding order, take the block scales from the first write, then code
        TensorPtr Kr = allocate(K->shape, *K), Vr = allocate(V->shape, *V);
        real1 *krp = device_ptr(*Kr, "forward"), *vrp = device_ptr(*Vr, "forward");
        HipDevice::check(weed_hip_apply_rotation_f32(hd, k_rot_dev->buffer, 4U, kv_shape, kp, K->offset, kv_str, krp, 0U, kv_str));
        HipDevice::check(weed_hip_apply_rotation_f32(hd, v_rot_dev->buffer, 4U, kv_shape, vp, V->offset, kv_str, vrp, 0U, kv_str));
        if (cache_len == 0U) {
            // sequential sums reproduce the reference bit for bit and are affordable for short first writes
            const int sequential = ((uint64_t)uB * Hkv * uT * hd <= (1U << 16)) ? 1 : 0;
            HipDevice::check(weed_hip_block_scale_f32(krp, 0U, kv_shape, kv_str, sequential, &k_qcache.block_scale));
            HipDevice::check(weed_hip_block_scale_f32(vrp, 0U, kv_shape, kv_str, sequential, &v_qcache.block_scale));
            HipDevice::check(weed_hip_kv_cache_set_scales(cache, k_qcache.block_scale, v_qcache.block_scale));
        }
        HipDevice::check(weed_hip_kv_encode_append(cache, 0, B, T, krp, 0U, kv_str, vrp, 0U, kv_str, 0));
    } else {
        HipDevice::check(weed_hip_kv_encode_append(cache, 0, B, T, kp, K->offset, kv_str, vp, V->offset, kv_str, 1));
    }
    const tcapint before = cache_len;
    cache_len += uT;
    k_qcache.outer = v_qcache.outer = uB * Hkv * cache_len;

    TensorPtr out = allocate({ uB, uT, Hq, hd }, *Q);
    real1 *qp = device_ptr(*Q, "forward"), *op = device_ptr(*out, "forward");
    const uint32_t q_str[3] = { 1U, uB * uT, uB * uT * Hq }; // (b, h, j) at a fixed t
    const int gqa = gqa_blocked ? WEED_HIP_GQA_BLOCKED : WEED_HIP_GQA_WEED;
    const uint32_t flags = WEED_HIP_ATTN_ROTATE_Q | WEED_HIP_ATTN_UNROTATE_OUT;
    if (T == 1) {
        HipDevice::check(weed_hip_kv_decode_attn(cache, num_heads, gqa, qp, Q->offset, q_str, op, 0U, q_str, flags));
        return out;
    }
    // the dense way builds [B, heads, T, L] score tensors, which 32-bit sizes and strides must be able to address
    const bool dense_fits = (uint64_t)uB * Hq * uT * cache_len <= (uint64_t)std::numeric_limits<tcapint>::max()
        && (uint64_t)uB * Hkv * cache_len * hd <= (uint64_t)std::numeric_limits<tcapint>::max();
    if (prefill_path == PREFILL_DENSE && !dense_fits) {
        throw std::invalid_argument("MultiHeadAttention::forward(): the dense prefill path would need score tensors of "
                                    "more elements than a 32-bit index can address; use the fused path");
    }
    if (dense_fits && (prefill_path == PREFILL_DENSE || (prefill_path == PREFILL_AUTO && dense_is_cheaper(uB, uT, cache_len)))) {
        // Long multi-token calls (prefill): the fused kernel serves one query position per launch, so beyond a few
        // positions it is cheaper to do what the reference does -- dequantise the cache once (still in the rotated
        // basis) and run dense ops: rotate Q, product, / sqrt(d), + mask, softmax, product, un-rotate
        // (multihead_attention.cpp:279-340).  The intermediates are private to this call, so they are laid out for
        // the device instead of column-major: head_dim (or the key position) is the contiguous dimension, the query
        // heads that share a KV head sit next to each other, and one batched product per (sequence, KV head) covers
        // the whole group without replicating K and V.
        const tcapint G = Hq / Hkv, L = cache_len, GT = G * uT;
        if ((uint64_t)uB * Hkv > 65535U) {
            throw std::invalid_argument("MultiHeadAttention::forward(): more than 65535 (sequence, KV head) pairs in a prefill");
        }
        TensorPtr K_deq = allocate_last_fastest({ uB, Hkv, L, hd }, *Q), V_deq = allocate_last_fastest({ uB, Hkv, L, hd }, *Q);
        HipDevice::check(weed_hip_kv_dequant(cache, 0, 0, B, 0, (int32_t)L, device_ptr(*K_deq, "forward"), 0U, K_deq->stride.data()));
        HipDevice::check(weed_hip_kv_dequant(cache, 1, 0, B, 0, (int32_t)L, device_ptr(*V_deq, "forward"), 0U, V_deq->stride.data()));
        // logical (B, Hkv, G, T, head_dim) views of Q and of the result: query head h = kv * G + g (blocked) or
        // g * Hkv + kv (Weed's kv = h % Hkv)
        const tcapint sH = Q->stride[2U];
        const tcapint shape5[5] = { uB, Hkv, G, uT, hd };
        const tcapint q5_str[5] = { Q->stride[0U], gqa_blocked ? G * sH : sH, gqa_blocked ? sH : Hkv * sH, Q->stride[1U],
            Q->stride[3U] };
        TensorPtr Q_rot = allocate_last_fastest({ uB, Hkv, G, uT, hd }, *Q);
        HipDevice::check(weed_hip_apply_rotation_f32(hd, k_rot_dev->buffer, 5U, shape5, qp, Q->offset, q5_str,
            device_ptr(*Q_rot, "forward"), 0U, Q_rot->stride.data()));
        // scores[b, kv, g*T + t, l] = q . k
        TensorPtr scores = allocate_last_fastest({ uB, Hkv, G, uT, L }, *Q);
        const tcapint pairs[2] = { uB, Hkv };
        const tcapint q_bs[2] = { Hkv * GT * hd, GT * hd }, kv_bs[2] = { Hkv * L * hd, L * hd }, s_bs[2] = { Hkv * GT * L, GT * L };
        HipDevice::check(weed_hip_matmul_batched_f32(pairs, GT, L, hd, device_ptr(*Q_rot, "forward"), 0U, hd, 1U, q_bs,
            device_ptr(*K_deq, "forward"), 0U, 1U, hd, kv_bs, device_ptr(*scores, "forward"), 0U, L, 1U, s_bs));
        TensorPtr inv = std::make_shared<Tensor>(real1(std::sqrt((real1)head_dim)), false, Q->storage->device,
            Q->storage->get_device_id());
        elementwise(WEED_HIP_EW_DIV, *scores, inv.get(), *scores, "MultiHeadAttention::forward");
        TensorPtr mask = Tensor::zeros({ uT, L }, false, false, DType::REAL, Q->storage->device);
        Weed::triu_fill(*mask, (real1)mask_val, before + 1U);
        elementwise(WEED_HIP_EW_ADD, *scores, mask.get(), *scores, "MultiHeadAttention::forward");
        TensorPtr weights = allocate_last_fastest({ uB, Hkv, G, uT, L }, *Q);
        HipDevice::check(weed_hip_softmax_f32(5U, scores->shape.data(), 4U, device_ptr(*scores, "forward"), 0U,
            scores->stride.data(), device_ptr(*weights, "forward"), 0U, weights->stride.data()));
        TensorPtr att = allocate_last_fastest({ uB, Hkv, G, uT, hd }, *Q);
        HipDevice::check(weed_hip_matmul_batched_f32(pairs, GT, hd, L, device_ptr(*weights, "forward"), 0U, L, 1U, s_bs,
            device_ptr(*V_deq, "forward"), 0U, hd, 1U, kv_bs, device_ptr(*att, "forward"), 0U, hd, 1U, q_bs));
        if (!v_rot_t_dev) {
            v_rot_t_dev = std::make_shared<GpuRealStorage>(v_rotation_trans);
        }
        // out is (B, T, H, head_dim) column-major like Q
        const tcapint oH = out->stride[2U];
        const tcapint o5_str[5] = { out->stride[0U], gqa_blocked ? G * oH : oH, gqa_blocked ? oH : Hkv * oH, out->stride[1U],
            out->stride[3U] };
        HipDevice::check(weed_hip_apply_rotation_f32(hd, v_rot_t_dev->buffer, 5U, shape5, device_ptr(*att, "forward"), 0U,
            att->stride.data(), op, 0U, o5_str));
        return out;
    }
    // causal attention: query position t sees the first before + t + 1 cached tokens of its sequence
    // The (position, head) pairs of a KV head are the rows of the fused kernel's tiles: one call serves up to 64
    // positions (a pass over the cache per tile of pairs), each masking the tokens after its own position.  Shapes
    // without matrix-core instances go position by position through the generic kernel.
    const tcapint per_call = matrix_core_shape() ? 64U : 1U;
    const uint32_t q_str4[4] = { Q->stride[0U], Q->stride[1U], Q->stride[2U], Q->stride[3U] };
    const uint32_t o_str4[4] = { out->stride[0U], out->stride[1U], out->stride[2U], out->stride[3U] };
    if (uT <= per_call) {
        // One call: its positions are the last uT cached tokens of every sequence, which is what the entry points
        // assume without a length array (no host-built lengths, no transfer, no wait for earlier launches).
        if (uT == 1U) {
            HipDevice::check(weed_hip_kv_decode_attn(cache, num_heads, gqa, qp, Q->offset, q_str, op, 0U, q_str, flags));
        } else {
            HipDevice::check(weed_hip_kv_decode_attn_chunk(cache, nullptr, (int32_t)uT, num_heads, gqa, qp, Q->offset,
                q_str4, op, 0U, o_str4, flags));
        }
        return out;
    }
    const size_t need = sizeof(int32_t) * (size_t)uB * uT;
    if (need > lens_cap) {
        if (lens_dev) {
            HipDevice::check(weed_hip_sync());
            (void)weed_hip_free(lens_dev);
            lens_dev = nullptr;
            lens_cap = 0U;
        }
        HipDevice::check(weed_hip_malloc(&lens_dev, need));
        lens_cap = need;
    }
    std::vector<int32_t> lens((size_t)uB * uT);
    for (tcapint t = 0U; t < uT; ++t) {
        std::fill(lens.begin() + (size_t)t * uB, lens.begin() + (size_t)(t + 1U) * uB, (int32_t)(before + t + 1U));
    }
    HipDevice::check(weed_hip_sync()); // earlier launches may still read the previous call's lengths
    HipDevice::check(weed_hip_memcpy_h2d(lens_dev, lens.data(), need));
    for (tcapint t = 0U; t < uT; t += per_call) {
        const tcapint n = std::min(per_call, uT - t);
        const int32_t *lens_t = static_cast<const int32_t *>(lens_dev) + (size_t)(t + n - 1U) * uB;
        if (n == 1U) {
            HipDevice::check(weed_hip_kv_decode_attn_prefix(cache, lens_t, num_heads, gqa, qp, Q->offset + t * Q->stride[1U],
                q_str, op, t * out->stride[1U], q_str, flags));
        } else {
            HipDevice::check(weed_hip_kv_decode_attn_chunk(cache, lens_t, (int32_t)n, num_heads, gqa, qp,
                Q->offset + t * Q->stride[1U], q_str4, op, t * out->stride[1U], o_str4, flags));
        }
    }
    return out;
}

// Whether the fused kernel's matrix-core instances serve this module's cache: head_dim up to 128 with fields of
// 2..5 bits (any pair) or of equal width 1, 6, 7 or 8; above 128 with fields of up to 4 bits.  Other shapes go
// through the generic kernel, one query position at a time.
bool MultiHeadAttention::matrix_core_shape() const
{
    const int wk = (k_bits ? k_bits : kv_quant_bits) + ((kv_coder == KV_LLOYDMAX && k_sign) ? 1 : 0);
    const int wv = (v_bits ? v_bits : kv_quant_bits) + ((kv_coder == KV_LLOYDMAX && v_sign) ? 1 : 0);
    const bool narrow = (wk >= 2 && wk <= 4 && wv >= 2 && wv <= 4) || (wk == 1 && wv == 1);
    if (head_dim > 128) {
        return narrow;
    }
    return narrow || (wk >= 2 && wk <= 5 && wv >= 2 && wv <= 5) || (wk == wv && wk >= 6 && wk <= 8);
}

// Rough device times of the two ways to serve T new tokens against L cached ones (measured on MI355X: a pass of the
// fused kernel costs about 55 us plus the packed bytes at 5 TB/s; the dense path is a dozen launches (200 us), writes
// and re-reads fp32 K and V, runs two batched fp32 products at 60 TFLOP/s and walks the [B, heads, T, L] scores seven
// times at 4 TB/s).
bool MultiHeadAttention::dense_is_cheaper(tcapint B, tcapint T, tcapint L) const
{
    const double Hkv = (double)num_kv_heads, Hq = (double)num_heads, hd = (double)head_dim;
    const double kb = (double)(k_bits ? k_bits : kv_quant_bits) + (k_sign ? 1.0 : 0.0);
    const double vb = (double)(v_bits ? v_bits : kv_quant_bits) + (v_sign ? 1.0 : 0.0);
    const double packed = (double)B * Hkv * (double)L * (hd * (kb + vb) / 8.0 + 8.0);
    // a pass serves one tile of (position, head) pairs: 16 rows, 8 above head_dim 128; the generic kernel takes one
    // position per pass at about a tenth of the rate
    const bool tiles = matrix_core_shape();
    const double tile_rows = head_dim > 128 ? 8.0 : 16.0;
    const double passes = tiles ? std::ceil((double)T * (Hq / Hkv) / tile_rows) : (double)T;
    const double fused_us = passes * (55.0 + packed / (tiles ? 5.0e6 : 0.5e6));
    const double deq_bytes = (double)B * Hkv * (double)L * hd * 4.0 * 2.0;
    const double flops = 2.0 * 2.0 * (double)B * Hq * (double)T * (double)L * hd;
    const double score_bytes = (double)B * Hq * (double)T * (double)L * 4.0 * 7.0;
    const double dense_us = 200.0 + deq_bytes / 3.0e6 + flops / 60.0e6 + score_bytes / 4.0e6;
    return dense_us < fused_us;
}

// Float cache or no cache: the reference's own sequence of dense ops (multihead_attention.cpp:279-340), each one a
// device op.  Returns (B, T, num_heads, head_dim).
TensorPtr MultiHeadAttention::forward_dense(TensorPtr Q, TensorPtr K, TensorPtr V, symint B, symint T)
{
    const tcapint hd = (tcapint)head_dim, Hkv = (tcapint)num_kv_heads;
    const tcapint uB = (tcapint)B, uT = (tcapint)T;
    Q = Tensor::transpose(Q, 1, 2); // [B, num_heads, T, head_dim]
    K = Tensor::transpose(K, 1, 2); // [B, kv_heads,  T, head_dim]
    V = Tensor::transpose(V, 1, 2);

    tcapint before = 0U;
    if (use_kv_cache) {
        if (!k_cache) {
            if (!max_seq_len) {
                max_seq_len = 2048U;
            }
            cache_len = 0U;
            k_cache = Tensor::zeros({ uB, Hkv, max_seq_len, hd }, false, false, DType::REAL, Q->storage->device);
            v_cache = Tensor::zeros({ uB, Hkv, max_seq_len, hd }, false, false, DType::REAL, Q->storage->device);
        }
        if (cache_len + uT > max_seq_len) {
            throw std::out_of_range("MultiHeadAttention::forward(): KV cache is full");
        }
        TensorPtr k_slot = Tensor::slice(k_cache, 2, cache_len, uT);
        TensorPtr v_slot = Tensor::slice(v_cache, 2, cache_len, uT);
        Weed::add_in_place(*k_slot, *K);
        Weed::add_in_place(*v_slot, *V);
        before = cache_len;
        cache_len += uT;
        K = Tensor::slice(k_cache, 2, 0U, cache_len);
        V = Tensor::slice(v_cache, 2, 0U, cache_len);
    }

    return Tensor::transpose(attend_dense(Q, K, V, before), 1, 2); // (B, T, H, head_dim)
}

// Dense causal attention as the reference spells it (multihead_attention.cpp:291-337): Q (B, H, T, hd), K and V
// (B, Hkv, T_k, hd) with the T new tokens last; query t sees keys 0 .. before + t.  Returns (B, H, T, hd).
TensorPtr MultiHeadAttention::attend_dense(TensorPtr Q, TensorPtr K, TensorPtr V, tcapint before)
{
    const tcapint hd = (tcapint)head_dim, Hkv = (tcapint)num_kv_heads, Hq = (tcapint)num_heads;
    const tcapint uB = Q->shape[0U], uT = Q->shape[2U];
    if (num_kv_heads < num_heads) {
        const tcapint groups = Hq / Hkv, T_k = K->shape[2U];
        TensorPtr K_rep = Tensor::zeros({ uB, Hq, T_k, hd }, false, false, DType::REAL, Q->storage->device);
        TensorPtr V_rep = Tensor::zeros({ uB, Hq, T_k, hd }, false, false, DType::REAL, Q->storage->device);
        if (gqa_blocked) {
            for (tcapint h = 0U; h < Hkv; ++h) {
                Weed::add_in_place(*Tensor::slice(K_rep, 1, h * groups, groups), *Tensor::slice(K, 1, h, 1U));
                Weed::add_in_place(*Tensor::slice(V_rep, 1, h * groups, groups), *Tensor::slice(V, 1, h, 1U));
            }
        } else {
            for (tcapint g = 0U; g < groups; ++g) {
                Weed::add_in_place(*Tensor::slice(K_rep, 1, g * Hkv, Hkv), *K);
                Weed::add_in_place(*Tensor::slice(V_rep, 1, g * Hkv, Hkv), *V);
            }
        }
        K = K_rep;
        V = V_rep;
    }

    TensorPtr scores = Q >> Tensor::transpose(K, -2, -1);
    scores = scores / real1(std::sqrt((real1)head_dim));
    if (uT > 1U) {
        const tcapint T_k = K->shape[2U];
        TensorPtr mask = Tensor::zeros({ uT, T_k }, false, false, DType::REAL, Q->storage->device);
        Weed::triu_fill(*mask, (real1)mask_val, before + 1U);
        scores = scores + mask;
    }
    TensorPtr weights = Tensor::softmax(scores, -1);
    return weights >> V;
}

// ---------------------------------------------------------------------------------------------------------
// norms, SwiGLU and the two modules that call the attention module
// ---------------------------------------------------------------------------------------------------------

RMSNorm::RMSNorm(const tcapint &hidden_size_, const symint &axis_, DeviceTag dtag)
    : Module(RMS_NORM_T)
    , axis(axis_)
    , hidden_size(hidden_size_)
{
    weight = std::make_shared<Parameter>(std::vector<real1>(hidden_size_, ONE_R1), std::vector<tcapint>{ hidden_size_ }, false, dtag);
}

TensorPtr RMSNorm::forward(const TensorPtr x)
{
    const symint ax = wrap_axis(axis, x->shape.size(), "RMSNorm::forward");
    if (x->shape[(size_t)ax] != hidden_size || weight->get_size() != hidden_size) {
        throw std::invalid_argument("Tensor shape mismatch in mul!"); // what the reference's `* weight` reports
    }
    validate_all_same_device({ x.get(), weight.get() }, "RMSNorm::forward");
    TensorPtr out = allocate(x->shape, *x);
    real1 *xp = device_ptr(*x, "RMSNorm::forward"), *wp = device_ptr(*weight, "RMSNorm::forward");
    real1 *op = device_ptr(*out, "RMSNorm::forward");
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_rms_norm_f32((uint32_t)x->shape.size(), x->shape.data(), (uint32_t)ax, xp, x->offset,
        x->stride.data(), wp, weight->offset, weight->stride.back(), FP_NORM_EPSILON, op, out->offset, out->stride.data()));
    return out;
}

LayerNorm::LayerNorm(const tcapint &f, const DeviceTag &dtag, const real1 &e, const int64_t &did)
    : Module(LAYERNORM_T)
    , features(f)
    , eps(e)
{
    gamma = std::make_shared<Parameter>(std::vector<real1>(f, ONE_R1), std::vector<tcapint>{ 1U, 1U, f }, true, dtag, did);
    beta = std::make_shared<Parameter>(std::vector<real1>(f, ZERO_R1), std::vector<tcapint>{ 1U, 1U, f }, true, dtag, did);
}

TensorPtr LayerNorm::forward(const TensorPtr x)
{
    if (x->shape.empty() || x->shape.back() != features || gamma->get_size() != features || beta->get_size() != features) {
        throw std::invalid_argument("Tensor shape mismatch in mul!");
    }
    validate_all_same_device({ x.get(), gamma.get(), beta.get() }, "LayerNorm::forward");
    TensorPtr out = allocate(x->shape, *x);
    real1 *xp = device_ptr(*x, "LayerNorm::forward"), *gp = device_ptr(*gamma, "LayerNorm::forward");
    real1 *bp = device_ptr(*beta, "LayerNorm::forward"), *op = device_ptr(*out, "LayerNorm::forward");
    WEED_DEVICE_LOCK();
    HipDevice::check(weed_hip_layer_norm_f32((uint32_t)x->shape.size(), x->shape.data(), (uint32_t)x->shape.size() - 1U, xp,
        x->offset, x->stride.data(), gp, gamma->offset, gamma->stride.back(), bp, beta->offset, beta->stride.back(), eps, op,
        out->offset, out->stride.data()));
    return out;
}

SwiGLU::SwiGLU(const tcapint &hidden_size_, const tcapint &intermediate_size_, DeviceTag dtag)
    : Module(SWIGLU_T)
    , hidden_size(hidden_size_)
    , intermediate_size(intermediate_size_)
{
    gate_proj = std::make_shared<Linear>(hidden_size, intermediate_size, false, true, DType::REAL, dtag);
    up_proj = std::make_shared<Linear>(hidden_size, intermediate_size, false, true, DType::REAL, dtag);
    down_proj = std::make_shared<Linear>(intermediate_size, hidden_size, false, true, DType::REAL, dtag);
    _register_params();
}

void SwiGLU::_register_params()
{
    param_vector.clear();
    for (const LinearPtr &l : { gate_proj, up_proj, down_proj }) {
        const std::vector<ParameterPtr> p = l->parameters();
        param_vector.insert(param_vector.end(), p.begin(), p.end());
    }
}

void SwiGLU::fuse_projections()
{
    if (gate_proj && up_proj) {
        place_side_by_side({ gate_proj, up_proj });
    }
}

TensorPtr SwiGLU::forward(const TensorPtr x)
{
    if (!gate_proj || !up_proj || !down_proj) {
        throw std::domain_error("SwiGLU::forward(): the module has no projections (default-constructed)");
    }
    const std::vector<TensorPtr> gu = forward_side_by_side({ gate_proj, up_proj }, x);
    TensorPtr gate = gu[0U], up = gu[1U];
    // SiLU(gate) * up
    TensorPtr activated = allocate(gate->shape, *gate);
    elementwise(WEED_HIP_EW_SILU_MUL, *gate, up.get(), *activated, "SwiGLU::forward");
    return down_proj->forward(activated);
}

TransformerEncoderLayer::TransformerEncoderLayer(const tcapint &d_model_, const tcapint &num_heads_, const tcapint &d_ff_,
    const DeviceTag &dtag, const ActivationFunctionType &afn, const int64_t &did)
    : Module(TRANSFORMER_ENCODER_LAYER_T)
    , d_model(d_model_)
    , d_ff(d_ff_)
    , num_heads(num_heads_)
    , self_attn(std::make_shared<MultiHeadAttention>(d_model_, num_heads_, num_heads_, 0U, dtag, nullptr, ZERO_R1, did))
    , ff1(std::make_shared<Linear>(d_model_, d_ff_, true, true, DType::REAL, dtag, did))
    , ff2(std::make_shared<Linear>(d_ff_, d_model_, true, true, DType::REAL, dtag, did))
    , norm1(std::make_shared<LayerNorm>(d_model_, dtag, FP_NORM_EPSILON, did))
    , norm2(std::make_shared<LayerNorm>(d_model_, dtag, FP_NORM_EPSILON, did))
{
    switch (afn) {
    case SIGMOID_FN:
        activation = std::make_shared<Sigmoid>();
        break;
    case TANH_FN:
        activation = std::make_shared<Tanh>();
        break;
    case RELU_FN:
        activation = std::make_shared<ReLU>();
        break;
    case SWIGLU_FN:
        // the reference puts a SwiGLU without projections here (transformer_encoder_layer.cpp:50-52), which cannot run
        throw std::invalid_argument("TransformerEncoderLayer: SWIGLU_FN has no projections to run between ff1 and ff2");
    case GELU_FN:
    default:
        activation = std::make_shared<GeLU>();
    }
    _register_params();
}

void TransformerEncoderLayer::_register_params()
{
    param_vector = self_attn->parameters();
    for (const std::vector<ParameterPtr> &q : { ff1->parameters(), ff2->parameters(), norm1->parameters(), norm2->parameters() }) {
        param_vector.insert(param_vector.end(), q.begin(), q.end());
    }
}

void TransformerEncoderLayer::fuse_projections() { self_attn->fuse_projections(); }

TensorPtr TransformerEncoderLayer::forward(const TensorPtr x)
{
    TensorPtr x1 = self_attn->forward(norm1->forward(x));
    x1 = x + x1;
    TensorPtr ff = ff2->forward(activation->forward(ff1->forward(norm2->forward(x1))));
    return x1 + ff;
}

QwenDecoderLayer::QwenDecoderLayer(const tcapint &d_model_, const tcapint &num_heads_, const tcapint &num_kv_heads_,
    const tcapint &d_ff_, const tcapint &max_seq_len, const real1_f &rope_base, const real1_f &, const int64_t &did)
    : Module(QWEN_DECODER_LAYER_T)
    , d_model(d_model_)
    , num_heads(num_heads_)
    , num_kv_heads(num_kv_heads_)
{
    // (the reference takes `eps` and never hands it on: RMSNorm always uses FP_NORM_EPSILON, rms_norm.hpp:35)
    const tcapint head_dim = d_model_ / num_heads_;
    RoPEPtr rope = std::make_shared<RoPE>(head_dim, max_seq_len, rope_base);
    self_attn = std::make_shared<MultiHeadAttention>(d_model_, num_heads_, num_kv_heads_, head_dim, DEFAULT_DEVICE, rope,
        ZERO_R1, did);
    mlp = std::make_shared<SwiGLU>(d_model_, d_ff_);
    input_layernorm = std::make_shared<RMSNorm>(d_model_, -1);
    post_attention_layernorm = std::make_shared<RMSNorm>(d_model_, -1);
    _register_params();
}

void QwenDecoderLayer::_register_params()
{
    param_vector.clear();
    for (const std::vector<ParameterPtr> &q : { self_attn->parameters(), mlp->parameters(), input_layernorm->parameters(),
             post_attention_layernorm->parameters() }) {
        param_vector.insert(param_vector.end(), q.begin(), q.end());
    }
}

void QwenDecoderLayer::fuse_projections()
{
    self_attn->fuse_projections();
    mlp->fuse_projections();
}

TensorPtr QwenDecoderLayer::forward(const TensorPtr x)
{
    // pre-norm + attention + residual
    TensorPtr h = self_attn->forward(input_layernorm->forward(x));
    h = h + x;
    // pre-norm + feed-forward + residual
    TensorPtr f = mlp->forward(post_attention_layernorm->forward(h));
    return f + h;
}

} // namespace Weed
