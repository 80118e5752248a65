// Checkpoint streams of the attention path: Storage, Parameter, Linear, RoPE, MultiHeadAttention, the norms and
// activations, SwiGLU, TransformerEncoderLayer, QwenDecoderLayer.
//
// The byte layout is the reference's at its default build widths (include/common/serializer.hpp,
// src/storage/storage.cpp:25-119, src/tensors/parameter.cpp:16-56, src/modules/module.cpp:53-260,
// src/modules/linear.cpp:109-118, src/modules/rope.cpp:100-106, src/modules/multihead_attention.cpp:358-375,
// include/modules/rms_norm.hpp:39-44, src/modules/layernorm.cpp:44-50, src/modules/swiglu.cpp:18-25,
// src/modules/transformer_encoder_layer.cpp:126-138, src/modules/qwen_decoder_layer.cpp:18-27):
//
//   Module      u32 module type
//   Linear      Module, u32 in_features, u32 out_features, Parameter weight, u8 has_bias, [Parameter bias]
//   RoPE        Module, u32 head_dim, u32 max_seq_len, f32 base
//   Attention   Module, f32 mask_val, i32 d_model, i32 num_heads, i32 num_kv_heads, i32 head_dim, u8 use_kv_cache,
//               i32 kv_quant_bits, Linear W_q, W_k, W_v, W_o, u8 has_rope, [RoPE]
//   ReLU, Sigmoid, Tanh, GeLU   Module (the tag alone)
//   RMSNorm     Module, i32 axis, u32 hidden_size, Parameter weight
//   LayerNorm   Module, u32 features, f32 eps, Parameter gamma, Parameter beta
//   SwiGLU      Module, u32 hidden_size, u32 intermediate_size, Linear gate_proj, up_proj, down_proj
//   Encoder layer   Module, u32 d_model, u32 d_ff, u32 num_heads, Attention, Linear ff1, ff2, LayerNorm norm1, norm2,
//               activation module
//   Qwen layer  Module, u32 d_model, u32 num_heads, u32 num_kv_heads, Attention, SwiGLU, RMSNorm input_layernorm,
//               RMSNorm post_attention_layernorm
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
    // A parameter that is a view of a larger storage (projections laid side by side, place_side_by_side) is written
    // as a compact copy of its own elements: the stream is the one the module wrote before it was moved.
    tcapint span = 1U;
    for (size_t i = 0U; i < shape.size(); ++i) {
        span += (shape[i] - 1U) * stride[i];
    }
    if (offset != 0U || storage->size != span) {
        std::shared_ptr<Tensor> self = std::make_shared<Tensor>(static_cast<const Tensor &>(*this));
        const TensorPtr own = Tensor::compact(self);
        Parameter copy;
        static_cast<Tensor &>(copy) = *own;
        copy.save(out);
        return;
    }
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

void RMSNorm::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_symint(os, axis);
    Serializer::write_tcapint(os, hidden_size);
    weight->save(os);
}

void LayerNorm::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, features);
    Serializer::write_real(os, eps);
    gamma->save(os);
    beta->save(os);
}

void SwiGLU::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, hidden_size);
    Serializer::write_tcapint(os, intermediate_size);
    gate_proj->save(os);
    up_proj->save(os);
    down_proj->save(os);
}

void TransformerEncoderLayer::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, d_model);
    Serializer::write_tcapint(os, d_ff);
    Serializer::write_tcapint(os, num_heads);
    self_attn->save(os);
    ff1->save(os);
    ff2->save(os);
    norm1->save(os);
    norm2->save(os);
    activation->save(os);
}

void QwenDecoderLayer::save(std::ostream &os) const
{
    Module::save(os);
    Serializer::write_tcapint(os, d_model);
    Serializer::write_tcapint(os, num_heads);
    Serializer::write_tcapint(os, num_kv_heads);
    self_attn->save(os);
    mlp->save(os);
    input_layernorm->save(os);
    post_attention_layernorm->save(os);
}

namespace {
// the sub-module a record names next, which must be of type T
template <typename T> std::shared_ptr<T> load_as(std::istream &is, const char *what)
{
    std::shared_ptr<T> m = std::dynamic_pointer_cast<T>(Module::load(is));
    if (!m) {
        throw std::runtime_error(std::string("module record: ") + what + " is not of the expected module type");
    }
    return m;
}
LinearPtr load_linear(std::istream &is) { return load_as<Linear>(is, "a projection"); }
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
    case RELU_T:
        return std::make_shared<ReLU>();
    case SIGMOID_T:
        return std::make_shared<Sigmoid>();
    case TANH_T:
        return std::make_shared<Tanh>();
    case GELU_T:
        return std::make_shared<GeLU>();
    case RMS_NORM_T: {
        RMSNormPtr r = std::make_shared<RMSNorm>();
        Serializer::read_symint(is, r->axis);
        Serializer::read_tcapint(is, r->hidden_size);
        r->weight = Parameter::load(is);
        return r;
    }
    case LAYERNORM_T: {
        LayerNormPtr l = std::make_shared<LayerNorm>();
        Serializer::read_tcapint(is, l->features);
        Serializer::read_real(is, l->eps);
        l->gamma = Parameter::load(is);
        l->beta = Parameter::load(is);
        return l;
    }
    case SWIGLU_T: {
        SwiGLUPtr g = std::make_shared<SwiGLU>();
        Serializer::read_tcapint(is, g->hidden_size);
        Serializer::read_tcapint(is, g->intermediate_size);
        g->gate_proj = load_linear(is);
        g->up_proj = load_linear(is);
        g->down_proj = load_linear(is);
        g->_register_params();
        return g;
    }
    case TRANSFORMER_ENCODER_LAYER_T: {
        TransformerEncoderLayerPtr t = std::make_shared<TransformerEncoderLayer>();
        Serializer::read_tcapint(is, t->d_model);
        Serializer::read_tcapint(is, t->d_ff);
        Serializer::read_tcapint(is, t->num_heads);
        t->self_attn = load_as<MultiHeadAttention>(is, "the attention of an encoder layer");
        t->ff1 = load_linear(is);
        t->ff2 = load_linear(is);
        t->norm1 = load_as<LayerNorm>(is, "norm1 of an encoder layer");
        t->norm2 = load_as<LayerNorm>(is, "norm2 of an encoder layer");
        t->activation = Module::load(is);
        t->_register_params();
        return t;
    }
    case QWEN_DECODER_LAYER_T: {
        QwenDecoderLayerPtr q = std::make_shared<QwenDecoderLayer>();
        Serializer::read_tcapint(is, q->d_model);
        Serializer::read_tcapint(is, q->num_heads);
        Serializer::read_tcapint(is, q->num_kv_heads);
        q->self_attn = load_as<MultiHeadAttention>(is, "the attention of a decoder layer");
        q->mlp = load_as<SwiGLU>(is, "the feed-forward block of a decoder layer");
        q->input_layernorm = load_as<RMSNorm>(is, "input_layernorm");
        q->post_attention_layernorm = load_as<RMSNorm>(is, "post_attention_layernorm");
        q->_register_params();
        return q;
    }
    default:
        throw std::domain_error("Module::load: module type " + std::to_string(tag) + " is not part of this build");
    }
}

// ---- the quantizer record (extension) ----
namespace {
constexpr uint32_t kQuantizerMagicV1 = 0x31515a57U; // "WZQ1": no tables
constexpr uint32_t kQuantizerMagic = 0x32515a57U;   // "WZQ2": the record below
void put_floats(std::ostream &os, const std::vector<real1> &v)
{
    Serializer::write_tcapint(os, (tcapint)v.size());
    for (const real1 &x : v) {
        Serializer::write_real(os, x);
    }
}
void get_floats(std::istream &is, std::vector<real1> &v, size_t most)
{
    tcapint n;
    Serializer::read_tcapint(is, n);
    if (n > most) {
        throw std::runtime_error("MultiHeadAttention::load_quantizer: implausible table size");
    }
    v.resize(n);
    for (real1 &x : v) {
        Serializer::read_real(is, x);
    }
}
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
        put_floats(os, *r);
    }
    // the Lloyd-Max tables that set_tables() installed, K side then V side: thresholds, levels, reconstruction
    // values; three empty lists stand for the built-in tables
    for (const CoderTables &t : custom_tables) {
        put_floats(os, t.bounds);
        put_floats(os, t.levels);
        put_floats(os, t.recon);
    }
}

void MultiHeadAttention::load_quantizer(std::istream &is)
{
    uint32_t magic;
    get(is, magic);
    if (magic != kQuantizerMagic && magic != kQuantizerMagicV1) {
        throw std::runtime_error("MultiHeadAttention::load_quantizer: not a quantizer record");
    }
    if (cache_len) {
        throw std::logic_error("MultiHeadAttention::load_quantizer: the cache already holds tokens; reset_cache() first");
    }
    if (k_qcache.dev) {
        // a live (still empty) device cache was made with the old settings: the next forward() makes a new one
        reset_cache();
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
    for (CoderTables &t : custom_tables) {
        t = CoderTables{};
    }
    if (magic == kQuantizerMagic) {
        for (int which = 0; which < 2; ++which) {
            CoderTables t;
            get_floats(is, t.bounds, 255U);
            get_floats(is, t.levels, 256U);
            get_floats(is, t.recon, 512U);
            if (!t.bounds.empty() || !t.levels.empty() || !t.recon.empty()) {
                set_tables(which, t.bounds, t.levels, t.recon); // checks the sizes against the code widths just read
            }
        }
    }
}

} // namespace Weed
