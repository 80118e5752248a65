// Host-side mirror of the part of Weed's C++ interface that sits on the quantized-KV attention path:
// Storage / Tensor (real, dense, forward only), the op entry points with their device switch, Linear,
// QuantizedKVCache and MultiHeadAttention, and the two modules that call it -- TransformerEncoderLayer and
// QwenDecoderLayer -- with the norms and activations they are made of.  Names, argument meaning and exception types
// follow the reference (include/tensors/tensor.hpp, include/storage/*.hpp, include/ops/*.hpp, include/modules/*.hpp);
// every computation goes to the device library behind
// include/weed_hip.h.  There is no CPU arithmetic here: a CPU-tagged tensor is a host container that can be filled,
// read and moved to the device, and an op handed one throws std::domain_error.
#pragma once

#include <cstdint>
#include <iosfwd>
#include <memory>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

struct weed_hip_kv_cache;

namespace Weed {

typedef uint32_t tcapint; // include/common/weed_types.hpp:48-66 at the default build width
typedef int32_t symint;
typedef float real1;
typedef float real1_f;
constexpr real1 ZERO_R1 = 0.0f;
constexpr real1 ONE_R1 = 1.0f;

enum DeviceTag { NONE_DEVICE = 0, DEFAULT_DEVICE = 1, CPU = 2, GPU = 3 }; // include/enums/device_tag.hpp
enum DType { NONE_DTYPE = 0, REAL = 1, COMPLEX = 2, INT = 3, DEFAULT_DTYPE = REAL }; // include/enums/dtype.hpp
// include/enums/storage_type.hpp (complex and sparse storages, tags 3, 4, 7, 8, are not part of this build)
enum StorageType { NONE_STORAGE_TYPE = 0, REAL_CPU_DENSE = 1, REAL_GPU_DENSE = 2, INT_CPU_DENSE = 5, INT_GPU_DENSE = 6 };
// include/enums/module_type.hpp: the tags a serialized module starts with.  Only the modules of this path can be
// written or read here; any other tag is reported by its number.
enum ModuleType {
    NONE_MODULE_TYPE = 0,
    LINEAR_T = 2,
    RELU_T = 3,
    SIGMOID_T = 4,
    TANH_T = 5,
    LAYERNORM_T = 7,
    MULTIHEAD_ATTENTION_T = 17,
    TRANSFORMER_ENCODER_LAYER_T = 18,
    GELU_T = 19,
    RMS_NORM_T = 30,
    ROPE_T = 31,
    SWIGLU_T = 32,
    QWEN_DECODER_LAYER_T = 33,
};
// include/enums/activation_function_type.hpp
enum ActivationFunctionType { NONE_FN = 0, SIGMOID_FN = 1, TANH_FN = 2, RELU_FN = 3, GELU_FN = 4, SWIGLU_FN = 5 };
// include/common/weed_types.hpp:213-214 at fp32: the epsilon both norms default to
constexpr real1 FP_NORM_EPSILON = 1.1920928955078125e-07f / 4.0f;

// include/common/serializer.hpp: fixed-width little-endian fields, written as the reference's default build writes
// them (tcapint and symint 32 bits, real1 and real1_f IEEE single, bool one byte, enums 32 bits).
struct Serializer {
    static void write_bool(std::ostream &out, const bool &x);
    static void read_bool(std::istream &in, bool &x);
    static void write_tcapint(std::ostream &out, const tcapint &x);
    static void read_tcapint(std::istream &in, tcapint &x);
    static void write_symint(std::ostream &out, const symint &x);
    static void read_symint(std::istream &in, symint &x);
    // Eight bytes.  The reference passes a 32-bit value by reference and writes eight bytes from its address
    // (serializer.hpp:51-56), so only the low four are defined: this writer sign-extends, the reader keeps the low four.
    static void write_int64(std::ostream &out, const symint &x);
    static void read_int64(std::istream &in, symint &x);
    static void write_real(std::ostream &out, const real1 &x);
    static void read_real(std::istream &in, real1 &x);
    static void write_real1_f(std::ostream &out, const real1_f &x);
    static void read_real1_f(std::istream &in, real1_f &x);
};

// include/devices/pool_item.hpp:32-40
struct bad_alloc : public std::bad_alloc {
    std::string m;
    explicit bad_alloc(std::string message)
        : m(std::move(message))
    {
    }
    const char *what() const noexcept override { return m.c_str(); }
};

// The one device behind every GPU storage and op (stands where GpuDevice + OCLEngine stand in the reference,
// include/devices/gpu_device.hpp, include/common/oclengine.hpp).  One HIP stream; entry points are serialised
// by `mutex`, as the reference serialises its queue (src/devices/gpu_device.cpp:195-203).
struct HipDevice {
    static HipDevice &Instance();
    std::recursive_mutex mutex;
    int64_t device_id;
    std::string name;
    // Block until everything queued has finished; a kernel failure surfaces here as std::runtime_error.
    void finish();
    // Translate a status code of the C ABI into the exception the reference would throw.
    static void check(int status);

private:
    HipDevice();
};

struct Storage;
typedef std::shared_ptr<Storage> StoragePtr;

// include/storage/storage.hpp:28-110
struct Storage : public std::enable_shared_from_this<Storage> {
    StorageType stype;
    DeviceTag device;
    DType dtype;
    tcapint size;

    Storage(StorageType stp, DeviceTag dtg, DType dtp, tcapint n);
    virtual ~Storage() {}
    virtual bool is_sparse() const { return false; }
    virtual tcapint get_sparse_size() const { return size; }
    virtual StoragePtr get_ptr() { return shared_from_this(); }
    virtual int64_t get_device_id() const { return -1; }
    virtual void FillZeros() = 0;
    virtual void FillOnes() = 0;
    virtual StoragePtr cpu() = 0;
    virtual StoragePtr gpu(int64_t did = -1) = 0;
    // src/storage/storage.cpp:25-30 plus the element loop of the real storages (cpu_real_storage.cpp:46-51,
    // gpu_real_storage.cpp:35-50): type tag, device id (8 bytes), size, then the elements.
    virtual void save(std::ostream &os) const;
    // src/storage/storage.cpp:32-119 for the two real dense types; a GPU storage is uploaded on load.
    static StoragePtr load(std::istream &is);
};

// include/storage/typed_storage.hpp:30-72 for T = real1
struct RealStorage : public Storage {
    using Storage::Storage;
    virtual real1 operator[](const tcapint &idx) const = 0;
    virtual void write(const tcapint &idx, const real1 &val) = 0;
    virtual void add(const tcapint &idx, const real1 &val) = 0;
    virtual void FillValue(const real1 &v) = 0;
};
typedef std::shared_ptr<RealStorage> RealStoragePtr;

// include/storage/cpu_real_storage.hpp
struct CpuRealStorage : public RealStorage {
    std::vector<real1> data;
    explicit CpuRealStorage(tcapint n);
    explicit CpuRealStorage(const std::vector<real1> &val);
    real1 operator[](const tcapint &idx) const override;
    void write(const tcapint &idx, const real1 &val) override;
    void add(const tcapint &idx, const real1 &val) override;
    void FillZeros() override;
    void FillOnes() override;
    void FillValue(const real1 &v) override;
    StoragePtr cpu() override { return get_ptr(); }
    StoragePtr gpu(int64_t did = -1) override; // uploads a copy (src/storage/cpu_real_storage.cpp:19-34)
};

// include/storage/gpu_real_storage.hpp, include/storage/gpu_storage.hpp:25-60: owns its device buffer
struct GpuRealStorage : public RealStorage {
    real1 *buffer;
    int64_t did;
    GpuRealStorage(tcapint n, int64_t did = -1);
    explicit GpuRealStorage(const std::vector<real1> &val, int64_t did = -1);
    ~GpuRealStorage() override;
    GpuRealStorage(const GpuRealStorage &) = delete;
    GpuRealStorage &operator=(const GpuRealStorage &) = delete;
    int64_t get_device_id() const override { return did; }
    real1 operator[](const tcapint &idx) const override; // blocking one-element read, as GpuDevice::GetReal
    void write(const tcapint &idx, const real1 &val) override;
    void add(const tcapint &idx, const real1 &val) override;
    void FillZeros() override;
    void FillOnes() override;
    void FillValue(const real1 &v) override;
    StoragePtr cpu() override; // new CpuRealStorage filled by a blocking read (src/storage/gpu_real_storage.cpp:18-23)
    StoragePtr gpu(int64_t = -1) override { return get_ptr(); }
};

// include/storage/typed_storage.hpp:30-72 for T = symint: the element type of symbol tables (token ids).
struct IntStorage : public Storage {
    using Storage::Storage;
    virtual symint operator[](const tcapint &idx) const = 0;
    virtual void write(const tcapint &idx, const symint &val) = 0;
    virtual void add(const tcapint &idx, const symint &val) = 0;
    virtual void FillValue(const symint &v) = 0;
    void save(std::ostream &os) const override; // header, then the elements as 32-bit integers (cpu_int_storage.cpp)
};

// include/storage/cpu_int_storage.hpp
struct CpuIntStorage : public IntStorage {
    std::vector<symint> data;
    explicit CpuIntStorage(tcapint n);
    explicit CpuIntStorage(const std::vector<symint> &val);
    symint operator[](const tcapint &idx) const override;
    void write(const tcapint &idx, const symint &val) override;
    void add(const tcapint &idx, const symint &val) override;
    void FillZeros() override;
    void FillOnes() override;
    void FillValue(const symint &v) override;
    StoragePtr cpu() override { return get_ptr(); }
    StoragePtr gpu(int64_t did = -1) override; // uploads a copy
};

// include/storage/gpu_int_storage.hpp, include/storage/gpu_storage.hpp:25-102: owns its device buffer; allocation,
// fills and the blocking transfers, which is all the reference does with integer storage on a device.  Element writes
// are refused as there (gpu_storage.hpp:88-94).
struct GpuIntStorage : public IntStorage {
    symint *buffer;
    int64_t did;
    GpuIntStorage(tcapint n, int64_t did = -1);
    explicit GpuIntStorage(const std::vector<symint> &val, int64_t did = -1);
    ~GpuIntStorage() override;
    GpuIntStorage(const GpuIntStorage &) = delete;
    GpuIntStorage &operator=(const GpuIntStorage &) = delete;
    int64_t get_device_id() const override { return did; }
    symint operator[](const tcapint &idx) const override; // blocking one-element read, as GpuDevice::GetInt
    void write(const tcapint &idx, const symint &val) override;
    void add(const tcapint &idx, const symint &val) override;
    void FillZeros() override;
    void FillOnes() override;
    void FillValue(const symint &v) override;
    StoragePtr cpu() override; // new CpuIntStorage filled by a blocking read (src/storage/gpu_int_storage.cpp:17-23)
    StoragePtr gpu(int64_t = -1) override { return get_ptr(); }
};

struct Tensor;
typedef std::shared_ptr<Tensor> TensorPtr;

// include/tensors/base_tensor.hpp + include/tensors/tensor.hpp, real dense tensors only.  Column-major: dimension 0
// is the contiguous one, dimensions of size 1 carry stride 0 (base_tensor.hpp:282-292).
struct Tensor {
    StoragePtr storage;
    std::vector<tcapint> shape;
    std::vector<tcapint> stride;
    tcapint offset = 0U;
    bool requires_grad = false; // kept for signature compatibility; there is no autograd on this path

    Tensor() {}
    Tensor(const std::vector<tcapint> &shp, const std::vector<tcapint> &str, const bool &rg = false,
        const bool &s = true, const DType &dtype = DType::REAL, const DeviceTag &dtag = DeviceTag::DEFAULT_DEVICE,
        const int64_t &did = -1);
    Tensor(const std::vector<real1> &val, const std::vector<tcapint> &shp, const bool &rg = false,
        const DeviceTag &dtag = DeviceTag::DEFAULT_DEVICE, const int64_t &did = -1);
    Tensor(const real1 &val, const bool &rg = false, const DeviceTag &dtag = DeviceTag::DEFAULT_DEVICE,
        const int64_t &did = -1);
    virtual ~Tensor() {}

    tcapint get_size() const;
    bool is_scalar() const;
    bool is_contiguous() const { return is_contiguous(shape, stride); }
    tcapint get_storage_index(const tcapint &idx) const; // base_tensor.hpp:123-142
    real1 get_item() const; // value of a one-element tensor (RealScalar::get_item)
    TensorPtr operator[](const tcapint &idx) const; // view with the LAST dimension fixed (tensor.cpp:277-293)
    std::vector<real1> to_vector() const; // logical elements in column-major order, read back from any device
    TensorPtr cast(const DeviceTag &dtag) const; // copy of the storage on the other side, same geometry

    static bool is_contiguous(const std::vector<tcapint> &shp, const std::vector<tcapint> &s);
    static std::vector<tcapint> full_contiguous_stride(const std::vector<tcapint> &shp);
    // element count in 64 bits; throws std::invalid_argument when it exceeds what tcapint can index
    static uint64_t checked_elements(const std::vector<tcapint> &shp);

    static TensorPtr zeros(const std::vector<tcapint> &shape, const bool &rg = false, const bool &s = true,
        const DType &dtype = DType::REAL, const DeviceTag &dtag = DeviceTag::DEFAULT_DEVICE, const int64_t &did = -1);
    static TensorPtr contiguous(const TensorPtr a);
    // `a` itself when its storage holds exactly its elements in order, else a copy that does
    static TensorPtr compact(const TensorPtr a);
    static TensorPtr reshape(const TensorPtr a, const std::vector<symint> &s);
    static TensorPtr transpose(const TensorPtr a);
    static TensorPtr transpose(const TensorPtr a, symint i, symint j);
    static TensorPtr slice(TensorPtr a, const int64_t &row);
    static TensorPtr slice(TensorPtr a, int64_t axis, const tcapint &start, const tcapint &length);
    static TensorPtr softmax(const TensorPtr x, symint axis);
    static TensorPtr sum(TensorPtr a, symint axis);
    static TensorPtr max(TensorPtr a, symint axis);
    static TensorPtr min(TensorPtr a, symint axis);
    static TensorPtr add(TensorPtr a, TensorPtr b);
    static TensorPtr sub(TensorPtr a, TensorPtr b);
    static TensorPtr mul(TensorPtr a, TensorPtr b);
    static TensorPtr div(TensorPtr a, TensorPtr b);
    static TensorPtr matmul(TensorPtr a, TensorPtr b);
    // src/tensors/tensor.cpp:682-693: sum along the axis, divided by its length; the axis stays with extent 1
    static TensorPtr mean(TensorPtr a, symint axis);
    // src/tensors/tensor.cpp:841-935: one elementwise kernel each (the reference composes gelu from eight ops)
    static TensorPtr relu(TensorPtr a);
    static TensorPtr sigmoid(TensorPtr a);
    static TensorPtr tanh(TensorPtr a);
    static TensorPtr gelu(const TensorPtr x);
};

TensorPtr operator+(TensorPtr left, TensorPtr right);
TensorPtr operator-(TensorPtr left, TensorPtr right);
TensorPtr operator*(TensorPtr left, TensorPtr right);
TensorPtr operator/(TensorPtr left, TensorPtr right);
TensorPtr operator/(TensorPtr left, real1 right);
TensorPtr operator*(real1 left, TensorPtr right);
TensorPtr operator>>(TensorPtr left, TensorPtr right); // matmul(left, right)
TensorPtr operator<<(TensorPtr right, TensorPtr left); // matmul(left, right)

// Op entry points (include/ops/*.hpp).  Each validates as the reference does and then switches on
// out.storage->device (src/ops/matmul.cpp:76-84): GPU launches the HIP kernel, anything else throws std::domain_error.
void matmul(const Tensor &a, const Tensor &b, Tensor &out); // src/ops/matmul.cpp:242-279
void softmax(const tcapint &index, const Tensor &a, Tensor &out); // src/ops/softmax.cpp:276-287
void reduce(const tcapint &index, const Tensor &a, Tensor &out); // src/ops/reduce.cpp:342-360
void max(const tcapint &index, const Tensor &a, Tensor &out); // src/ops/reduce.cpp:362-373
void min(const tcapint &index, const Tensor &a, Tensor &out); // src/ops/reduce.cpp:375-386
void add(const Tensor &a, const Tensor &b, Tensor &out); // src/ops/commuting.cpp
void mul(const Tensor &a, const Tensor &b, Tensor &out);
void sub(const Tensor &a, const Tensor &b, Tensor &out); // src/ops/sub.cpp
void div(const Tensor &a, const Tensor &b, Tensor &out); // src/ops/div.cpp:17-20
void add_in_place(Tensor &a, const Tensor &b); // src/ops/in_place.cpp:17-25
void triu_fill(Tensor &a, const real1 &val, const tcapint diagonal = 1); // src/ops/triu_fill.cpp:42-59
void relu(const Tensor &a, Tensor &out); // src/ops/real_unary.cpp:485-497
void sigmoid(const Tensor &a, Tensor &out);
void tanh(const Tensor &a, Tensor &out);

struct Parameter : public Tensor { // include/tensors/parameter.hpp
    using Tensor::Tensor;
    // src/tensors/parameter.cpp:16-56: device id, offset, rank, (shape, stride) pairs, storage.  As in the reference,
    // save() first sets the extent of every stride-0 dimension to 1.
    void save(std::ostream &out);
    static std::shared_ptr<Parameter> load(std::istream &in);
};
typedef std::shared_ptr<Parameter> ParameterPtr;

// include/modules/module.hpp, the members this path uses
struct Module {
    ModuleType mtype;
    explicit Module(ModuleType t = NONE_MODULE_TYPE)
        : mtype(t)
    {
    }
    virtual ~Module() {}
    // src/modules/module.cpp:53-56: the type tag; the inheriting struct writes the rest.
    virtual void save(std::ostream &os) const;
    // src/modules/module.cpp:58-304 for the tags of ModuleType above; any other tag throws std::domain_error.
    static std::shared_ptr<Module> load(std::istream &is);
    virtual TensorPtr forward(const TensorPtr x) = 0;
    virtual std::vector<ParameterPtr> parameters() { return {}; }
    virtual void train() {}
    virtual void eval() {}
    virtual void set_max_kv_seq_len(tcapint) {}
    virtual void reset_cache() {}
};

// include/modules/linear.hpp:20-41, src/modules/linear.cpp:86-100
struct Linear : public Module {
    tcapint in_features;
    tcapint out_features;
    ParameterPtr weight; // (in_features, out_features)
    ParameterPtr bias; // (1, out_features) or null

    Linear()
        : Module(LINEAR_T)
        , in_features(0U)
        , out_features(0U)
    {
    }
    Linear(tcapint in_f, tcapint out_f, bool use_bias = true, bool init_rand = true, DType dtype = DType::REAL,
        DeviceTag device = DeviceTag::DEFAULT_DEVICE, int64_t device_id = -1);
    TensorPtr forward(const TensorPtr x) override;
    std::vector<ParameterPtr> parameters() override;
    void save(std::ostream &os) const override; // src/modules/linear.cpp:109-118
};
typedef std::shared_ptr<Linear> LinearPtr;

// Linear modules that read the same input and whose weights (in_features x out_features, a column per output) lie
// side by side in one storage, their biases in another, are applied with ONE product: the outputs of the first
// module, then those of the second, ... are consecutive columns of one result.  No counterpart in the reference,
// whose attention and SwiGLU modules launch one product per projection (Q, K, V; gate, up); at decode time the
// small ones cost a launch and a pass over half-empty compute units each.
// place_side_by_side(): moves the modules' weights and biases into such storages.  The Parameter objects stay the
//   same (lists of parameters held elsewhere remain valid), the values are copied; all modules need the same
//   in_features, device and bias-or-not.  A module saved afterwards writes a compact copy of its own weight, so the
//   stream is the same as before.
// forward_side_by_side(): the modules' outputs for x, in one launch when they lie side by side, else one by one.
void place_side_by_side(const std::vector<LinearPtr> &linears);
std::vector<TensorPtr> forward_side_by_side(const std::vector<LinearPtr> &linears, const TensorPtr x);

// The packed K and V rows of one attention module live in ONE device object (include/weed_hip.h); the two
// QuantizedKVCache members of the module are views of its two halves.
struct DeviceKVCache {
    weed_hip_kv_cache *handle = nullptr;
    tcapint n_seq = 0U, n_kv_heads = 0U, head_dim = 0U, max_tokens = 0U;
    DeviceKVCache(int mode, tcapint n_seq_, tcapint n_kv_heads_, tcapint head_dim_, tcapint max_tokens_, int k_bits,
        int v_bits, int k_sign, int v_sign);
    ~DeviceKVCache();
    DeviceKVCache(const DeviceKVCache &) = delete;
    DeviceKVCache &operator=(const DeviceKVCache &) = delete;
};
typedef std::shared_ptr<DeviceKVCache> DeviceKVCachePtr;

// include/modules/multihead_attention.hpp:22-36.  Rows live on the device.  Row r is token r % max_tokens of
// (sequence, kv head) pair r / max_tokens; a stand-alone cache made with allocate() is a single pair, so its rows
// are simply 0 .. max_outer-1.  Rows are append-only per pair: write_row(r) must name the next free row (the
// reference ORs new codes into old bits, src/modules/multihead_attention.cpp:58, so it cannot rewrite a row
// either).
struct QuantizedKVCache {
    std::vector<symint> packed; // Weed's int32 words of the rows written so far, refreshed by sync_packed()
    real1 block_scale = ONE_R1;
    tcapint outer = 0U; // rows written so far (stand-alone cache)
    tcapint d = 0U;
    tcapint max_outer = 0U;
    int bits = 0;
    DeviceKVCachePtr dev; // shared with the sibling cache inside a module
    int which = 0; // 0: the K half of `dev`, 1: the V half

    int values_per_word() const { return (int)(sizeof(symint) * 8) / bits; }
    void allocate(const tcapint max_outer_, const tcapint d_, const int bits_);
    void write_row(const tcapint row, const real1 *vals);
    void read_row(const tcapint row, real1 *vals) const;
    void sync_packed();
};

enum KVCoder { KV_UNIFORM = 0, KV_LLOYDMAX = 1 };

// include/modules/rope.hpp, src/modules/rope.cpp: rotary position embedding.  The tables are built on the host with
// the reference's fp32 arithmetic (rope.cpp:18-51) and live on the device; forward() is one fused kernel.
// forward(x, pos0) is an extension: token t of x uses position pos0 + t (the reference always starts at 0, which is
// only right for a call that begins a sequence).
struct RoPE : public Module {
    tcapint head_dim;
    tcapint max_seq_len;
    real1_f base;
    TensorPtr cos_table; // [max_seq_len, head_dim]
    TensorPtr sin_table; // [max_seq_len, head_dim]

    RoPE(const tcapint &head_dim_, const tcapint &max_seq_len_ = 2048U, const real1_f &base_ = 10000.0f,
        DeviceTag dtag = DEFAULT_DEVICE);
    void _build_tables(DeviceTag dtag);
    TensorPtr forward(const TensorPtr x) override { return forward(x, 0U); }
    TensorPtr forward(const TensorPtr x, tcapint pos0); // x: [B, H, T, head_dim], any strides
    void apply(const Tensor &x, Tensor &out, tcapint pos0); // the same into a given (possibly strided) output
    void save(std::ostream &os) const override; // src/modules/rope.cpp:100-106: the tables are rebuilt on load
};
typedef std::shared_ptr<RoPE> RoPEPtr;

// include/modules/multihead_attention.hpp:41-173.  Differences, all deliberate:
//  * W_k / W_v project to num_kv_heads * head_dim features, so grouped-query attention works with the stock
//    constructor (the reference builds d_model x d_model and needs them swapped by hand);
//  * tokens are appended in logical order, so prefill followed by decode steps is consistent (the reference's row
//    order only works for a single call);
//  * the causal mask honours the cache offset, and set_max_kv_seq_len() survives the first forward();
//  * RoPE, when present, is applied at the tokens' true positions (cache_len onwards), and max_seq_len defaults to
//    the RoPE table length as in the reference (cpp:173);
//  * rotation_seed makes the rotations reproducible (0 = draw a seed from std::random_device like the reference);
//    rotations already present in k_rotation / v_rotation at the first forward() are used as given;
//  * kv_coder selects the reference's uniform coder (default) or the Lloyd-Max coder with k_bits / v_bits / sign
//    bits; kv_quant_bits serves both K and V in uniform mode as in the reference.
struct MultiHeadAttention : public Module {
    symint d_model;
    symint num_heads;
    symint num_kv_heads;
    symint head_dim;
    real1_f mask_val;

    LinearPtr W_q;
    LinearPtr W_k;
    LinearPtr W_v;
    LinearPtr W_o;

    RoPEPtr rope; // applied to Q and K before the cache, at position cache_len (the reference: always position 0)

    bool use_kv_cache;
    TensorPtr k_cache; // float cache (kv_quant_bits == 0)
    TensorPtr v_cache;
    tcapint cache_len = 0U;
    tcapint max_seq_len = 0U;

    int kv_quant_bits = 0;
    std::vector<real1> k_rotation;
    std::vector<real1> v_rotation;
    QuantizedKVCache k_qcache;
    QuantizedKVCache v_qcache;
    std::vector<real1> v_rotation_trans;

    // extensions (see above)
    KVCoder kv_coder = KV_UNIFORM;
    int k_bits = 0, v_bits = 0; // 0: use kv_quant_bits
    bool k_sign = false, v_sign = false;
    bool gqa_blocked = false; // false: kv head = q head % num_kv_heads, the reference's mapping (cpp:291-311)
    // How a call with several new tokens attends over the quantised cache.  FUSED: groups of up to 16 / (heads per KV
    // head) positions per pass of the fused kernel over the packed rows.  DENSE: what the reference does -- dequantise
    // the cache once, then dense products, mask, softmax (multihead_attention.cpp:259-340).  AUTO picks by estimated
    // cost: short chunks against a long context go FUSED, a long prefill goes DENSE.
    enum PrefillPath { PREFILL_AUTO = 0, PREFILL_FUSED = 1, PREFILL_DENSE = 2 };
    PrefillPath prefill_path = PREFILL_AUTO;
    uint32_t rotation_seed = 0U;

    std::vector<ParameterPtr> param_vector;

    MultiHeadAttention(tcapint d_model_, tcapint num_heads_, tcapint num_kv_heads_ = 0, tcapint head_dim_ = 0U,
        DeviceTag dtag = DEFAULT_DEVICE, RoPEPtr r = nullptr, real1_f mask_val_ = ZERO_R1, const int64_t did = -1,
        const bool _use_kv_cache = true, int kv_quant_bits_ = 4, bool use_bias = true);

    // What Module::load builds on (multihead_attention.hpp: the reference's default constructor): no projections yet.
    MultiHeadAttention();
    // src/modules/multihead_attention.cpp:358-375, byte for byte the reference's stream: mask value, the four sizes,
    // use_kv_cache, kv_quant_bits, the four projections, the RoPE flag and module.  Neither the reference nor this
    // stream holds the cached tokens.
    void save(std::ostream &os) const override;
    // Extension, a separate record that a caller may write after save(): what the stream above lacks to make a
    // reloaded module encode and decode identically -- coder, bit widths, sign bits, head mapping, rotation seed,
    // max_seq_len, the two block scales and the two rotations (empty before the first forward()).
    // Since version 2 of the record also the Lloyd-Max tables of either side when set_tables() replaced them.
    void save_quantizer(std::ostream &os) const;
    void load_quantizer(std::istream &is);
    // Replace the built-in Lloyd-Max tables of the K side (which = 0) or the V side (1): 2^bits - 1 thresholds, 2^bits
    // levels, 2^(bits + sign) reconstruction values (weed_hip_kv_cache_set_tables).  Takes effect for the tokens coded
    // afterwards: call it before the first forward(), or after reset_cache().  The tables survive reset_cache() and
    // travel in the quantizer record.
    void set_tables(int which, const std::vector<real1> &bounds, const std::vector<real1> &levels,
        const std::vector<real1> &recon);
    struct CoderTables {
        std::vector<real1> bounds, levels, recon;
    };
    CoderTables custom_tables[2]; // empty vectors: the built-in tables

    std::vector<ParameterPtr> parameters() override { return param_vector; }
    void set_max_kv_seq_len(tcapint m) override { max_seq_len = m; }
    void reset_cache() override;
    TensorPtr forward(const TensorPtr x) override;
    // The Q, K and V projections as one product from now on (place_side_by_side; results agree to rounding).
    void fuse_projections();
    // PREFILL_AUTO's rule for B sequences, T new tokens and L cached ones (the new ones included): true when
    // dequantising once and attending densely is estimated cheaper than the passes of the fused kernel
    bool dense_is_cheaper(tcapint B, tcapint T, tcapint L) const;
    bool matrix_core_shape() const; // whether the fused kernel's matrix-core instances serve this module's cache

private:
    TensorPtr forward_quantized(TensorPtr Q, TensorPtr K, TensorPtr V, symint B, symint T);
    TensorPtr forward_dense(TensorPtr Q, TensorPtr K, TensorPtr V, symint B, symint T);
    TensorPtr attend_dense(TensorPtr Q, TensorPtr K, TensorPtr V, tcapint before);
    std::shared_ptr<GpuRealStorage> k_rot_dev, v_rot_dev, v_rot_t_dev; // device copies of the rotations
    void *lens_dev = nullptr; // int32 prefix lengths for multi-token calls
    size_t lens_cap = 0U;

public:
    ~MultiHeadAttention() override;
};
typedef std::shared_ptr<MultiHeadAttention> MultiHeadAttentionPtr;

// include/modules/relu.hpp, sigmoid.hpp, tanh.hpp, gelu.hpp: activation functions as modules (their stream is the tag
// alone).
struct ReLU : public Module {
    ReLU()
        : Module(RELU_T)
    {
    }
    TensorPtr forward(const TensorPtr x) override { return Tensor::relu(x); }
};
struct Sigmoid : public Module {
    Sigmoid()
        : Module(SIGMOID_T)
    {
    }
    TensorPtr forward(const TensorPtr x) override { return Tensor::sigmoid(x); }
};
struct Tanh : public Module {
    Tanh()
        : Module(TANH_T)
    {
    }
    TensorPtr forward(const TensorPtr x) override { return Tensor::tanh(x); }
};
struct GeLU : public Module {
    GeLU()
        : Module(GELU_T)
    {
    }
    TensorPtr forward(const TensorPtr x) override { return Tensor::gelu(x); }
};

// include/modules/rms_norm.hpp: x / sqrt(mean(x^2, axis) + eps) * weight.  forward() is one kernel
// (weed_hip_rms_norm_f32) where the reference chains seven elementwise ops and an axis sum.
struct RMSNorm : public Module {
    symint axis;
    tcapint hidden_size;
    ParameterPtr weight; // (hidden_size), ones

    RMSNorm()
        : Module(RMS_NORM_T)
        , axis(-1)
        , hidden_size(0U)
    {
    }
    RMSNorm(const tcapint &hidden_size_, const symint &axis_ = -1, DeviceTag dtag = DEFAULT_DEVICE);
    std::vector<ParameterPtr> parameters() override { return { weight }; }
    TensorPtr forward(const TensorPtr x) override;
    void save(std::ostream &os) const override; // rms_norm.hpp:39-44
};
typedef std::shared_ptr<RMSNorm> RMSNormPtr;

// include/modules/layernorm.hpp, src/modules/layernorm.cpp:29-50: normalisation over the last dimension, then
// gamma (ones) and beta (zeros), both of shape (1, 1, features).  forward() is one kernel (weed_hip_layer_norm_f32).
struct LayerNorm : public Module {
    tcapint features;
    real1 eps;
    ParameterPtr gamma;
    ParameterPtr beta;

    LayerNorm()
        : Module(LAYERNORM_T)
        , features(0U)
        , eps(FP_NORM_EPSILON)
    {
    }
    LayerNorm(const tcapint &f, const DeviceTag &dtag = DeviceTag::DEFAULT_DEVICE, const real1 &e = FP_NORM_EPSILON,
        const int64_t &did = -1);
    TensorPtr forward(const TensorPtr x) override;
    std::vector<ParameterPtr> parameters() override { return { gamma, beta }; }
    void save(std::ostream &os) const override;
};
typedef std::shared_ptr<LayerNorm> LayerNormPtr;

// include/modules/swiglu.hpp: down_proj(gate_proj(x) * sigmoid(gate_proj(x)) * up_proj(x)), three bias-free Linear
// modules.  The gate is one elementwise kernel (WEED_HIP_EW_SILU_MUL).  Unlike the reference's constructor, this one
// registers the projections' parameters right away (the reference only does so when a module is loaded).
struct SwiGLU : public Module {
    tcapint hidden_size;
    tcapint intermediate_size;
    LinearPtr gate_proj;
    LinearPtr up_proj;
    LinearPtr down_proj;
    std::vector<ParameterPtr> param_vector;

    SwiGLU()
        : Module(SWIGLU_T)
        , hidden_size(0U)
        , intermediate_size(0U)
    {
    }
    SwiGLU(const tcapint &hidden_size_, const tcapint &intermediate_size_, DeviceTag dtag = DEFAULT_DEVICE);
    void _register_params();
    std::vector<ParameterPtr> parameters() override { return param_vector; }
    TensorPtr forward(const TensorPtr x) override;
    // The gate and up projections as one product from now on (place_side_by_side).
    void fuse_projections();
    void save(std::ostream &os) const override; // src/modules/swiglu.cpp:18-25
};
typedef std::shared_ptr<SwiGLU> SwiGLUPtr;

// include/modules/transformer_encoder_layer.hpp, src/modules/transformer_encoder_layer.cpp:24-139: pre-norm block
// x1 = x + attn(norm1(x)); out = x1 + ff2(act(ff1(norm2(x1)))).  The reference's forward() also moves its sub-modules
// between host and device around every step (cpp:64-121); here everything lives on the device, so that is left out.
struct TransformerEncoderLayer : public Module {
    tcapint d_model;
    tcapint d_ff;
    tcapint num_heads;
    MultiHeadAttentionPtr self_attn;
    LinearPtr ff1;
    LinearPtr ff2;
    LayerNormPtr norm1;
    LayerNormPtr norm2;
    std::shared_ptr<Module> activation;
    std::vector<ParameterPtr> param_vector;

    TransformerEncoderLayer()
        : Module(TRANSFORMER_ENCODER_LAYER_T)
        , d_model(0U)
        , d_ff(0U)
        , num_heads(0U)
    {
    }
    TransformerEncoderLayer(const tcapint &d_model_, const tcapint &num_heads_, const tcapint &d_ff_,
        const DeviceTag &dtag = DEFAULT_DEVICE, const ActivationFunctionType &afn = GELU_FN, const int64_t &did = -1);
    void _register_params();
    std::vector<ParameterPtr> parameters() override { return param_vector; }
    void set_max_kv_seq_len(tcapint m) override { self_attn->set_max_kv_seq_len(m); }
    void reset_cache() override { self_attn->reset_cache(); }
    TensorPtr forward(const TensorPtr x) override;
    void fuse_projections(); // the attention module's
    void save(std::ostream &os) const override;
};
typedef std::shared_ptr<TransformerEncoderLayer> TransformerEncoderLayerPtr;

// include/modules/qwen_decoder_layer.hpp: h = x + attn(rms1(x)); out = h + mlp(rms2(h)), with rotary positions, grouped
// query heads and bias-carrying projections in the attention as the reference's constructor builds them (hpp:37-50).
struct QwenDecoderLayer : public Module {
    tcapint d_model;
    tcapint num_heads;
    tcapint num_kv_heads;
    MultiHeadAttentionPtr self_attn;
    SwiGLUPtr mlp;
    RMSNormPtr input_layernorm;
    RMSNormPtr post_attention_layernorm;
    std::vector<ParameterPtr> param_vector;

    QwenDecoderLayer()
        : Module(QWEN_DECODER_LAYER_T)
        , d_model(0U)
        , num_heads(0U)
        , num_kv_heads(0U)
    {
    }
    QwenDecoderLayer(const tcapint &d_model_, const tcapint &num_heads_, const tcapint &num_kv_heads_, const tcapint &d_ff_,
        const tcapint &max_seq_len = 2048U, const real1_f &rope_base = 10000.0f, const real1_f &eps = 1e-6f,
        const int64_t &did = -1);
    void _register_params();
    std::vector<ParameterPtr> parameters() override { return param_vector; }
    void set_max_kv_seq_len(tcapint m) override { self_attn->set_max_kv_seq_len(m); }
    void reset_cache() override { self_attn->reset_cache(); }
    TensorPtr forward(const TensorPtr x) override;
    void fuse_projections(); // the attention module's and the SwiGLU's
    void save(std::ostream &os) const override; // src/modules/qwen_decoder_layer.cpp:18-27
};
typedef std::shared_ptr<QwenDecoderLayer> QwenDecoderLayerPtr;

} // namespace Weed
