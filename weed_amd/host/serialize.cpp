// Checkpoint streams of the attention path: Storage, Parameter, Linear, RoPE, MultiHeadAttention.
//
// The byte layout is the reference's at its default build widths (include/common/serializer.hpp,
// src/storage/storage.cpp:25-119, src/tensors/parameter.cpp:16-56, src/modules/module.cpp:53-260,
// src/modules/linear.cpp:109-118, src/modules/rope.cpp:100-106, src/modules/multihead_attention.cpp:358-375):
//
//   Module      u32 module type
//   Linear      Module, u32 in_features, u32 out_features, Parameter weight, u8 has_bias, [Parameter bias]
//   RoPE        Module, u32 head_dim, u32 max_seq_len, f32 base
//   Attention   Module, f32 mask_val, i32 d_model, i32 num_heads, i32 num_kv_heads, i32 head_dim, u8 use_kv_cache,
//               i32 kv_quant_bits, Linear W_q, W_k, W_v, W_o, u8 has_rope, [RoPE]
//   Parameter   i32 device id, u32 offset, u32 rank, rank x (u32 shape, u32 stride), Storage
//   Storage     u32 storage type, 8 bytes device id (low four defined), u32 size, size x f32
//
// All fields little-endian, no padding.  The reference has no test or fixture of these streams, so what pins this
// file is the layout above checked against hand-assembled bytes, and round trips.
#include "weed.hpp"

#include <cstring>
#include <istream>
#include <ostream>
#include <stdexcept>

namespace Weed {

namespace {
template <typename T> void put(std::ostream &out, const T &x)
{
    char b[sizeof(T)];
    std::memcpy(b, &x, sizeof(T));
    out.write(b, sizeof(T));
    if (!out) {
        throw std::runtime_error("checkpoint stream: write failed");
    }
}
template <typename T> void get(std::istream &in, T &x)
{
    char b[sizeof(T)];
    in.read(b, sizeof(T));
    if (in.gcount() != (std::streamsize)sizeof(T)) {
        throw std::runtime_error("checkpoint stream: unexpected end of data");
    }
    std::memcpy(&x, b, sizeof(T));
}
static_assert(sizeof(bool) == 1 && sizeof(real1) == 4 && sizeof(tcapint) == 4 && sizeof(symint) == 4, "field widths");
} // namespace

void Serializer::write_bool(std::ostream &out, const bool &x) { put<uint8_t>(out, x ? 1U : 0U); }
void Serializer::read_bool(std::istream &in, bool &x)
{
    uint8_t b;
    get(in, b);
    x = b != 0U;
}
void Serializer::write_tcapint(std::ostream &out, const tcapint &x) { put(out, x); }
void Serializer::read_tcapint(std::istream &in, tcapint &x) { get(in, x); }
void Serializer::write_symint(std::ostream &out, const symint &x) { put(out, x); }
void Serializer::read_symint(std::istream &in, symint &x) { get(in, x); }
void Serializer::write_int64(std::ostream &out, const symint &x) { put<int64_t>(out, (int64_t)x); }
void Serializer::read_int64(std::istream &in, symint &x)
{
    uint64_t v;
    get(in, v);
    x = (symint)(uint32_t)(v & 0xffffffffULL);
}
void Serializer::write_real(std::ostream &out, const real1 &x) { put(out, x); }
void Serializer::read_real(std::istream &in, real1 &x) { get(in, x); }
void Serializer::write_real1_f(std::ostream &out, const real1_f &x) { put(out, x); }
void Serializer::read_real1_f(std::istream &in, real1_f &x) { get(in, x); }

// ---- Storage ----
void Storage::save(std::ostream &os) const
{
    put<uint32_t>(os, (uint32_t)stype);
    Serializer::write_int64(os, (symint)get_device_id());
    Serializer::write_tcapint(os, size);
    // the elements, through a host copy when they live on the device
    StoragePtr host = const_cast<Storage *>(this)->cpu();
    const CpuRealStorage *c = dynamic_cast<const CpuRealStorage *>(host.get());
    if (!c || c->data.size() != size) {
        throw std::domain_error("Storage::save: only real dense storage is part of this build");
    }
    for (tcapint i = 0U; i < size; ++i) {
        Serializer::write_real(os, c->data[i]);
    }
}

// Integer storage: the same header, then the elements as 32-bit integers (src/storage/cpu_int_storage.cpp,
// src/storage/gpu_int_storage.cpp:24-39).
void IntStorage::save(std::ostream &os) const
{
    put<uint32_t>(os, (uint32_t)stype);
    Serializer::write_int64(os, (symint)get_device_id());
    Serializer::write_tcapint(os, size);
    StoragePtr host = const_cast<IntStorage *>(this)->cpu();
    const CpuIntStorage *c = dynamic_cast<const CpuIntStorage *>(host.get());
    if (!c || c->data.size() != size) {
        throw std::domain_error("IntStorage::save: host copy failed");
    }
    for (tcapint i = 0U; i < size; ++i) {
        Serializer::write_symint(os, c->data[i]);
    }
}

StoragePtr Storage::load(std::istream &is)
{
    uint32_t tag;
    get(is, tag);
    symint did;
    Serializer::read_int64(is, did);
    tcapint size;
    Serializer::read_tcapint(is, size);
    if (tag == (uint32_t)INT_CPU_DENSE || tag == (uint32_t)INT_GPU_DENSE) {
        std::vector<symint> v(size);
        for (tcapint i = 0U; i < size; ++i) {
            Serializer::read_symint(is, v[i]);
        }
        if (tag == (uint32_t)INT_CPU_DENSE) {
            return std::make_shared<CpuIntStorage>(v);
        }
        return std::make_shared<GpuIntStorage>(v, (int64_t)did);
    }
    if (tag != (uint32_t)REAL_CPU_DENSE && tag != (uint32_t)REAL_GPU_DENSE) {
        // complex and sparse storages (tags 3, 4, 7, 8) exist in the reference and not here
        throw std::domain_error("Can't recognize StorageType in Storage::load!");
    }
    std::vector<real1> v(size);
    for (tcapint i = 0U; i < size; ++i) {
        Serializer::read_real(is, v[i]);
    }
    if (tag == (uint32_t)REAL_CPU_DENSE) {
        return std::make_shared<CpuRealStorage>(v);
    }
    return std::make_shared<GpuRealStorage>(v, (int64_t)did);
}

// ---- Parameter ----
void Parameter::save(std::ostream &out)
{
    Serializer::write_symint(out, (symint)storage->get_device_id());
    for (size_t i = 0U; i < stride.size(); ++i) {
        if (!stride[i]) {
            shape[i] = 1U;
        }
    }
    Serializer::write_tcapint(out, offset);
    Serializer::write_tcapint(out, (tcapint)shape.size());
    for (size_t i = 0U; i < shape.size(); ++i) {
        Serializer::write_tcapint(out, shape[i]);
        Serializer::write_tcapint(out, stride[i]);
    }
    storage->save(out);
}

ParameterPtr Parameter::load(std::istream &in)
{
    symint did;
    Serializer::read_symint(in, did);
    (void)did; // the storage record carries it again
    tcapint offset, rank;
    Serializer::read_tcapint(in, offset);
    Serializer::read_tcapint(in, rank);
    if (rank > 64U) {
        throw std::runtime_error("Parameter::load: implausible rank, not a parameter record");
    }
    ParameterPtr p = std::make_shared<Parameter>();
    p->shape.resize(rank);
    p->stride.resize(rank);
    for (tcapint i = 0U; i < rank; ++i) {
        Serializer::read_tcapint(in, p->shape[i]);
        Serializer::read_tcapint(in, p->stride[i]);
    }
    p->storage = Storage::load(in);
    // the reference's loader leaves the offset at zero (parameter.cpp:48-52); a view into a larger storage keeps it
    p->offset = offset;
    p->requires_grad = true;
    // every element the geometry can reach must exist
    tcapint last = offset;
    for (tcapint i = 0U; i < rank; ++i) {
        if (!p->shape[i]) {
            throw std::runtime_error("Parameter::load: empty dimension");
        }
        last += (p->shape[i] - 1U) * p->stride[i];
    }
    if (last >= p->storage->size) {
        throw std::runtime_error("Parameter::load: geometry exceeds the stored elements");
    }
    return p;
}

// ---- modules ----
void Module::save(std::ostream &os) const { put<uint32_t>(os, (uint32_t)mtype); }

void Linear::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, in_features);
    Serializer::write_tcapint(os, out_features);
    weight->save(os);
    Serializer::write_bool(os, !!bias);
    if (bias) {
        bias->save(os);
    }
}

void RoPE::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, head_dim);
    Serializer::write_tcapint(os, max_seq_len);
    Serializer::write_real1_f(os, base);
}

void MultiHeadAttention::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_real1_f(os, mask_val);
    Serializer::write_symint(os, d_model);
    Serializer::write_symint(os, num_heads);
    Serializer::write_symint(os, num_kv_heads);
    Serializer::write_symint(os, head_dim);
    Serializer::write_bool(os, use_kv_cache);
    Serializer::write_symint(os, (symint)kv_quant_bits);
    W_q->save(os);
    W_k->save(os);
    W_v->save(os);
    W_o->save(os);
    Serializer::write_bool(os, (bool)rope);
    if (rope) {
        rope->save(os);
    }
}

namespace {
LinearPtr load_linear(std::istream &is)
{
    LinearPtr l = std::dynamic_pointer_cast<Linear>(Module::load(is));
    if (!l) {
        throw std::runtime_error("MultiHeadAttention record: a projection is not a Linear module");
    }
    return l;
}
} // namespace

std::shared_ptr<Module> Module::load(std::istream &is)
{
    uint32_t tag;
    get(is, tag);
    switch (tag) {
    case LINEAR_T: {
        LinearPtr l = std::make_shared<Linear>();
        Serializer::read_tcapint(is, l->in_features);
        Serializer::read_tcapint(is, l->out_features);
        l->weight = Parameter::load(is);
        bool is_bias;
        Serializer::read_bool(is, is_bias);
        if (is_bias) {
            l->bias = Parameter::load(is);
        }
        return l;
    }
    case ROPE_T: {
        tcapint hd, msl;
        real1_f base;
        Serializer::read_tcapint(is, hd);
        Serializer::read_tcapint(is, msl);
        Serializer::read_real1_f(is, base);
        return std::make_shared<RoPE>(hd, msl, base); // builds the tables
    }
    case MULTIHEAD_ATTENTION_T: {
        MultiHeadAttentionPtr m = std::make_shared<MultiHeadAttention>();
        Serializer::read_real1_f(is, m->mask_val);
        Serializer::read_symint(is, m->d_model);
        Serializer::read_symint(is, m->num_heads);
        Serializer::read_symint(is, m->num_kv_heads);
        Serializer::read_symint(is, m->head_dim);
        Serializer::read_bool(is, m->use_kv_cache);
        symint bits = 0;
        Serializer::read_symint(is, bits);
        m->kv_quant_bits = (int)bits;
        m->W_q = load_linear(is);
        m->W_k = load_linear(is);
        m->W_v = load_linear(is);
        m->W_o = load_linear(is);
        bool has_rope;
        Serializer::read_bool(is, has_rope);
        if (has_rope) {
            m->rope = std::dynamic_pointer_cast<RoPE>(Module::load(is));
            if (!m->rope) {
                throw std::runtime_error("MultiHeadAttention record: the position module is not a RoPE");
            }
        }
        for (const LinearPtr &l : { m->W_q, m->W_k, m->W_v, m->W_o }) {
            const std::vector<ParameterPtr> p = l->parameters();
            m->param_vector.insert(m->param_vector.end(), p.begin(), p.end());
        }
        return m;
    }
    default:
        throw std::domain_error("Module::load: module type " + std::to_string(tag) + " is not part of this build");
    }
}

// ---- the quantizer record (extension) ----
namespace {
constexpr uint32_t kQuantizerMagic = 0x31515a57U; // "WZQ1"
}

void MultiHeadAttention::save_quantizer(std::ostream &os) const
{
    put<uint32_t>(os, kQuantizerMagic);
    Serializer::write_symint(os, (symint)kv_coder);
    Serializer::write_symint(os, (symint)k_bits);
    Serializer::write_symint(os, (symint)v_bits);
    Serializer::write_bool(os, k_sign);
    Serializer::write_bool(os, v_sign);
    Serializer::write_bool(os, gqa_blocked);
    Serializer::write_tcapint(os, rotation_seed);
    Serializer::write_tcapint(os, max_seq_len);
    Serializer::write_real(os, k_qcache.block_scale);
    Serializer::write_real(os, v_qcache.block_scale);
    for (const std::vector<real1> *r : { &k_rotation, &v_rotation }) {
        Serializer::write_tcapint(os, (tcapint)r->size());
        for (const real1 &x : *r) {
            Serializer::write_real(os, x);
        }
    }
}

void MultiHeadAttention::load_quantizer(std::istream &is)
{
    uint32_t magic;
    get(is, magic);
    if (magic != kQuantizerMagic) {
        throw std::runtime_error("MultiHeadAttention::load_quantizer: not a quantizer record");
    }
    if (cache_len) {
        throw std::logic_error("MultiHeadAttention::load_quantizer: the cache already holds tokens; reset_cache() first");
    }
    symint coder, kb, vb;
    Serializer::read_symint(is, coder);
    Serializer::read_symint(is, kb);
    Serializer::read_symint(is, vb);
    if ((coder != KV_UNIFORM && coder != KV_LLOYDMAX) || kb < 0 || kb > 8 || vb < 0 || vb > 8) {
        throw std::runtime_error("MultiHeadAttention::load_quantizer: implausible coder settings");
    }
    kv_coder = (KVCoder)coder;
    k_bits = (int)kb;
    v_bits = (int)vb;
    Serializer::read_bool(is, k_sign);
    Serializer::read_bool(is, v_sign);
    Serializer::read_bool(is, gqa_blocked);
    Serializer::read_tcapint(is, rotation_seed);
    Serializer::read_tcapint(is, max_seq_len);
    Serializer::read_real(is, k_qcache.block_scale);
    Serializer::read_real(is, v_qcache.block_scale);
    const tcapint want = (tcapint)(head_dim * head_dim);
    for (std::vector<real1> *r : { &k_rotation, &v_rotation }) {
        tcapint n;
        Serializer::read_tcapint(is, n);
        if (n != 0U && n != want) {
            throw std::runtime_error("MultiHeadAttention::load_quantizer: rotation size does not match head_dim");
        }
        r->resize(n);
        for (real1 &x : *r) {
            Serializer::read_real(is, x);
        }
    }
}

} // namespace Weed
