// Tests of the host C++ mirror, written the way the reference writes its own (test/tests.cpp): tensors are built
// with std::make_shared<Tensor>(values, shape, ...), ops are called through Tensor:: / operators, and results are
// read back through storage.  Cases marked `needs_gpu = false` exercise host logic only and run anywhere; the rest
// run every computation on the device and compare with the CPU checker (oracle/) or with closed forms.
//
// Usage: test_host_mirror [--no-gpu] [name-substring]
#include "weed.hpp"

#include "weed_oracle.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <sstream>
#include <vector>

using namespace Weed;

namespace {

struct Case {
    const char *name;
    bool needs_gpu;
    std::function<void()> body;
};
std::vector<Case> &cases()
{
    static std::vector<Case> c;
    return c;
}
struct Registrar {
    Registrar(const char *n, bool g, std::function<void()> b) { cases().push_back({ n, g, std::move(b) }); }
};
int failures = 0;

#define TEST_CASE(name, needs_gpu)                                                                                     \
    static void name();                                                                                                \
    static Registrar reg_##name(#name, needs_gpu, name);                                                               \
    static void name()

#define REQUIRE(cond)                                                                                                  \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            std::printf("    FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                          \
            ++failures;                                                                                                \
        }                                                                                                              \
    } while (0)

#define EPSILON 0.01f // test/tests.cpp:30
#define REQUIRE_FLOAT(A, B) REQUIRE(std::fabs((double)(A) - (double)(B)) < EPSILON)

#define REQUIRE_THROWS_AS(expr, type)                                                                                  \
    do {                                                                                                               \
        bool caught = false;                                                                                           \
        try {                                                                                                          \
            (void)(expr);                                                                                              \
        } catch (const type &) {                                                                                       \
            caught = true;                                                                                             \
        } catch (...) {                                                                                                \
        }                                                                                                              \
        if (!caught) {                                                                                                 \
            std::printf("    FAILED %s:%d: %s did not throw %s\n", __FILE__, __LINE__, #expr, #type);                  \
            ++failures;                                                                                                \
        }                                                                                                              \
    } while (0)

#define R(v) real1(v)
const DeviceTag TEST_DTAG = DeviceTag::GPU;

real1 get_real(const TensorPtr &t) { return t->get_item(); }

std::vector<real1> gaussian(size_t n, uint32_t seed, real1 scale = 1.0f)
{
    std::mt19937 rng(seed);
    std::normal_distribution<real1> dist(0.0f, 1.0f);
    std::vector<real1> v(n);
    for (real1 &x : v) {
        x = scale * dist(rng);
    }
    return v;
}

// The attention tolerance: |got - want| <= max(1e-4, 1e-3 |want|)
bool attn_close(const std::vector<real1> &got, const std::vector<double> &want, double *worst = nullptr)
{
    bool ok = got.size() == want.size();
    double w = 0.0;
    for (size_t i = 0; ok && i < got.size(); ++i) {
        const double err = std::fabs((double)got[i] - want[i]);
        w = std::max(w, err);
        if (!(err <= std::max(1e-4, 1e-3 * std::fabs(want[i])))) {
            ok = false;
        }
    }
    if (worst) {
        *worst = w;
    }
    return ok;
}

// --------------------------------------------------------------------------------------------------------------------
// host logic (no device)
// --------------------------------------------------------------------------------------------------------------------

TEST_CASE(test_column_major_geometry, false)
{
    // test/tests.cpp:1214-1218: element [r, c] of a 2x3 tensor is at index r + c*nrows
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(1), R(2), R(3), R(4), R(5), R(6) },
        std::vector<tcapint>{ 2, 3 }, false, DeviceTag::CPU);
    REQUIRE(x->stride == (std::vector<tcapint>{ 1U, 2U }));
    REQUIRE(x->get_storage_index(3U) == 3U);
    REQUIRE(get_real((*(*x)[2])[1]) == R(6)); // operator[] fixes the LAST index first
    REQUIRE(get_real((*(*x)[0])[1]) == R(2));
    TensorPtr t = Tensor::transpose(x);
    REQUIRE(t->shape == (std::vector<tcapint>{ 3U, 2U }));
    REQUIRE(t->stride == (std::vector<tcapint>{ 2U, 1U }));
    REQUIRE(!t->is_contiguous());
    REQUIRE(t->to_vector() == (std::vector<real1>{ 1, 3, 5, 2, 4, 6 }));
    TensorPtr s = Tensor::slice(x, 1, 1U, 2U);
    REQUIRE(s->offset == 2U);
    REQUIRE(s->to_vector() == (std::vector<real1>{ 3, 4, 5, 6 }));
    TensorPtr row = Tensor::slice(x, 1);
    REQUIRE(row->to_vector() == (std::vector<real1>{ 2, 4, 6 }));
    // size-1 dimensions carry stride 0 (include/tensors/base_tensor.hpp:282-292)
    REQUIRE(Tensor::full_contiguous_stride({ 1U, 4U, 1U, 3U }) == (std::vector<tcapint>{ 0U, 1U, 0U, 4U }));
    REQUIRE_THROWS_AS(x->get_storage_index(6U), std::invalid_argument);
    REQUIRE_THROWS_AS((*x)[3], std::invalid_argument);
}

TEST_CASE(test_reshape_rules, false)
{
    TensorPtr x = std::make_shared<Tensor>(
        std::vector<real1>{ 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11 }, std::vector<tcapint>{ 2, 6 }, false, DeviceTag::CPU);
    TensorPtr y = Tensor::reshape(x, { 2, -1, 2 });
    REQUIRE(y->shape == (std::vector<tcapint>{ 2U, 3U, 2U }));
    REQUIRE(y->storage == x->storage); // a contiguous tensor is re-viewed, not copied
    REQUIRE(y->to_vector() == x->to_vector());
    REQUIRE_THROWS_AS(Tensor::reshape(x, { -1, -1 }), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::reshape(x, { 5, -1 }), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::reshape(x, { 5, 2 }), std::invalid_argument);
    REQUIRE_THROWS_AS(std::make_shared<Tensor>(std::vector<real1>{ 1, 2, 3 }, std::vector<tcapint>{ 2, 2 }, false, DeviceTag::CPU),
        std::invalid_argument);
    REQUIRE_THROWS_AS(std::make_shared<CpuRealStorage>(0U), std::invalid_argument);
}

TEST_CASE(test_shapes_beyond_32_bit_indices_are_refused, false)
{
    // 3 * 32 * 8192 * 8192 = 3 * 2^31 elements (the score tensor of a three-sequence 8192-token prefill at 32 heads)
    // wraps to 2^31 in 32-bit arithmetic; 2 * ... wraps to 0.  Both must be refused before any storage exists.
    const std::vector<tcapint> three{ 3U, 32U, 8192U, 8192U }, two{ 2U, 32U, 8192U, 8192U };
    REQUIRE_THROWS_AS(Tensor::checked_elements(three), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::checked_elements(two), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::full_contiguous_stride(three), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::zeros(three, false, false, DType::REAL, DeviceTag::CPU), std::invalid_argument);
    REQUIRE_THROWS_AS(Tensor::zeros(two, false, false, DType::REAL, DeviceTag::CPU), std::invalid_argument);
    REQUIRE(Tensor::checked_elements({ 65535U, 65537U }) == 4294967295ULL); // the largest count that still fits
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ 0, 1, 2, 3 }, std::vector<tcapint>{ 2, 2 }, false, DeviceTag::CPU);
    REQUIRE_THROWS_AS(Tensor::reshape(x, { 65536, 65536 }), std::invalid_argument);
}

TEST_CASE(test_cpu_tensors_do_not_compute, false)
{
    // there is no CPU arithmetic in this build: an op handed host tensors must say so, never fall back
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(2), R(3) }, std::vector<tcapint>{ 1, 2 }, false, DeviceTag::CPU);
    TensorPtr y = std::make_shared<Tensor>(std::vector<real1>{ R(4), R(5) }, std::vector<tcapint>{ 2, 1 }, false, DeviceTag::CPU);
    REQUIRE_THROWS_AS(x >> y, std::domain_error);
    REQUIRE_THROWS_AS(Tensor::softmax(x, 1), std::domain_error);
    REQUIRE_THROWS_AS(Tensor::sum(x, 1), std::domain_error);
    REQUIRE_THROWS_AS(x + x, std::domain_error);
    QuantizedKVCache qc;
    real1 v[32] = { 0 };
    REQUIRE_THROWS_AS(qc.write_row(0U, v), std::domain_error);
    REQUIRE_THROWS_AS(qc.read_row(0U, v), std::domain_error);
}

// --------------------------------------------------------------------------------------------------------------------
// the reference's op tests, on the device (forward values; there is no autograd here)
// --------------------------------------------------------------------------------------------------------------------

TEST_CASE(test_real_matmul, true)
{
    // test/tests.cpp:1020-1041
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(2), R(3) }, std::vector<tcapint>{ 1, 2 }, false, TEST_DTAG);
    TensorPtr y = std::make_shared<Tensor>(std::vector<real1>{ R(4), R(5) }, std::vector<tcapint>{ 2, 1 }, false, TEST_DTAG);
    TensorPtr z = x >> y;
    REQUIRE(get_real((*z)[0]) == R(23));

    x = std::make_shared<Tensor>(std::vector<real1>{ R(2), R(3) }, std::vector<tcapint>{ 2, 1 }, false, TEST_DTAG);
    y = std::make_shared<Tensor>(std::vector<real1>{ R(4), R(5) }, std::vector<tcapint>{ 1, 2 }, false, TEST_DTAG);
    z = x >> y;
    REQUIRE(get_real((*(*z)[0])[0]) == R(8));
    REQUIRE(get_real((*(*z)[0])[1]) == R(12));
    REQUIRE(get_real((*(*z)[1])[0]) == R(10));
    REQUIRE(get_real((*(*z)[1])[1]) == R(15));
    z = y << x; // same product, operands swapped
    REQUIRE(get_real((*(*z)[1])[1]) == R(15));
}

TEST_CASE(test_matmul_2x3_3x2, true)
{
    // operands of test/tests.cpp:1327-1340 (column-major); C = A.B = [[76, 103], [100, 136]]
    TensorPtr A = std::make_shared<Tensor>(
        std::vector<real1>{ R(1), R(2), R(3), R(4), R(5), R(6) }, std::vector<tcapint>{ 2, 3 }, true, TEST_DTAG);
    TensorPtr B = std::make_shared<Tensor>(
        std::vector<real1>{ R(7), R(8), R(9), R(10), R(11), R(12) }, std::vector<tcapint>{ 3, 2 }, true, TEST_DTAG);
    TensorPtr C = A >> B;
    REQUIRE(C->to_vector() == (std::vector<real1>{ 76, 100, 103, 136 }));
    // a transposed view is a valid operand: B^T.A^T = C^T
    TensorPtr Ct = Tensor::transpose(B) >> Tensor::transpose(A);
    REQUIRE(Ct->to_vector() == (std::vector<real1>{ 76, 103, 100, 136 }));
    REQUIRE_THROWS_AS(A >> A, std::invalid_argument);
    TensorPtr host = A->cast(DeviceTag::CPU);
    REQUIRE_THROWS_AS(host >> B, std::invalid_argument); // device mismatch is reported before anything runs
}

TEST_CASE(test_softmax_forward, true)
{
    // test/tests.cpp:1110-1171
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(1), R(2), R(3) }, std::vector<tcapint>{ 3 }, false, TEST_DTAG);
    TensorPtr y = Tensor::softmax(x, 0);
    RealStorage *ys = static_cast<RealStorage *>(y->storage.get());
    REQUIRE_FLOAT((real1_f)(*ys)[0] + (real1_f)(*ys)[1] + (real1_f)(*ys)[2], 1.0f);

    x = std::make_shared<Tensor>(std::vector<real1>{ R(1), R(3), R(2) }, std::vector<tcapint>{ 3 }, false, TEST_DTAG);
    y = Tensor::softmax(x, 0);
    ys = static_cast<RealStorage *>(y->storage.get());
    REQUIRE((real1_f)(*ys)[1] > (real1_f)(*ys)[2]);
    REQUIRE((real1_f)(*ys)[2] > (real1_f)(*ys)[0]);

    x = std::make_shared<Tensor>(std::vector<real1>{ R(1000), R(1001), R(1002) }, std::vector<tcapint>{ 3 }, false, TEST_DTAG);
    y = Tensor::softmax(x, 0);
    ys = static_cast<RealStorage *>(y->storage.get());
    const real1_f sum = (real1_f)(*ys)[0] + (real1_f)(*ys)[1] + (real1_f)(*ys)[2];
    REQUIRE(std::isfinite(sum));
    REQUIRE_FLOAT(sum, 1.0f);

    x = std::make_shared<Tensor>(std::vector<real1>{ R(2), R(2), R(2) }, std::vector<tcapint>{ 3 }, false, TEST_DTAG);
    y = Tensor::softmax(x, 0);
    ys = static_cast<RealStorage *>(y->storage.get());
    REQUIRE_FLOAT((real1_f)(*ys)[0], 1.0f / 3.0f);
    REQUIRE_FLOAT((real1_f)(*ys)[2], 1.0f / 3.0f);

    x = std::make_shared<Tensor>(std::vector<real1>{ R(0), R(1) }, std::vector<tcapint>{ 2 }, false, TEST_DTAG);
    y = Tensor::softmax(x, 0);
    ys = static_cast<RealStorage *>(y->storage.get());
    const real1_f denom = 1.0f + std::exp(1.0f);
    REQUIRE(std::fabs((*ys)[0] - 1.0f / denom) < 1e-6f);
    REQUIRE(std::fabs((*ys)[1] - std::exp(1.0f) / denom) < 1e-6f);
}

TEST_CASE(test_softmax_axis1, true)
{
    // test/tests.cpp:1206-1221
    TensorPtr x = std::make_shared<Tensor>(
        std::vector<real1>{ R(1), R(2), R(3), R(4), R(5), R(6) }, std::vector<tcapint>{ 2, 3 }, false, TEST_DTAG);
    TensorPtr y = Tensor::softmax(x, 1);
    RealStorage *ys = static_cast<RealStorage *>(y->storage.get());
    REQUIRE_FLOAT((real1_f)(*ys)[0] + (real1_f)(*ys)[2] + (real1_f)(*ys)[4], 1.0f);
    REQUIRE_FLOAT((real1_f)(*ys)[1] + (real1_f)(*ys)[3] + (real1_f)(*ys)[5], 1.0f);
    TensorPtr z = Tensor::softmax(x, -1); // negative axes count from the end
    REQUIRE(z->to_vector() == y->to_vector());
}

TEST_CASE(test_axis_reductions, true)
{
    // test/tests.cpp:177-228
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(1), R(1) }, std::vector<tcapint>{ 2 }, true, TEST_DTAG);
    REQUIRE(get_real(Tensor::sum(x, 0U)) == R(2));
    x = std::make_shared<Tensor>(std::vector<real1>{ R(0), R(1) }, std::vector<tcapint>{ 2 }, true, TEST_DTAG);
    REQUIRE(get_real(Tensor::max(x, 0U)) == R(1));
    REQUIRE(get_real(Tensor::min(x, 0U)) == R(0));
    // a 2x3 matrix along both axes
    x = std::make_shared<Tensor>(
        std::vector<real1>{ R(1), R(2), R(3), R(4), R(5), R(6) }, std::vector<tcapint>{ 2, 3 }, false, TEST_DTAG);
    REQUIRE(Tensor::sum(x, 0)->to_vector() == (std::vector<real1>{ 3, 7, 11 }));
    REQUIRE(Tensor::sum(x, 1)->to_vector() == (std::vector<real1>{ 9, 12 }));
    REQUIRE(Tensor::max(x, 1)->to_vector() == (std::vector<real1>{ 5, 6 }));
    REQUIRE(Tensor::min(Tensor::transpose(x), 0)->to_vector() == (std::vector<real1>{ 1, 2 }));
}

TEST_CASE(test_elementwise_and_storage_round_trip, true)
{
    TensorPtr a = std::make_shared<Tensor>(
        std::vector<real1>{ R(1), R(2), R(3), R(4), R(5), R(6) }, std::vector<tcapint>{ 2, 3 }, false, TEST_DTAG);
    TensorPtr b = std::make_shared<Tensor>(std::vector<real1>{ R(10), R(20), R(30) }, std::vector<tcapint>{ 1, 3 }, false, TEST_DTAG);
    REQUIRE((a + b)->to_vector() == (std::vector<real1>{ 11, 12, 23, 24, 35, 36 }));
    REQUIRE((a - b)->to_vector() == (std::vector<real1>{ -9, -8, -17, -16, -25, -24 }));
    REQUIRE((a * b)->to_vector() == (std::vector<real1>{ 10, 20, 60, 80, 150, 180 }));
    REQUIRE((a / R(2))->to_vector() == (std::vector<real1>{ 0.5f, 1, 1.5f, 2, 2.5f, 3 }));
    REQUIRE((R(2) * a)->to_vector() == (std::vector<real1>{ 2, 4, 6, 8, 10, 12 }));
    REQUIRE(Tensor::contiguous(Tensor::transpose(a))->to_vector() == (std::vector<real1>{ 1, 3, 5, 2, 4, 6 }));
    Weed::add_in_place(*a, *b);
    REQUIRE(a->to_vector() == (std::vector<real1>{ 11, 12, 23, 24, 35, 36 }));
    TensorPtr m = Tensor::zeros({ 3U, 4U }, false, false, DType::REAL, TEST_DTAG);
    Weed::triu_fill(*m, R(-7));
    REQUIRE(m->to_vector() == (std::vector<real1>{ 0, 0, 0, -7, 0, 0, -7, -7, 0, -7, -7, -7 }));
    // storage: device -> host copy is a new object, host -> device likewise (src/storage/gpu_real_storage.cpp:18-23)
    StoragePtr host = a->storage->cpu();
    REQUIRE(host->device == DeviceTag::CPU);
    REQUIRE(host != a->storage);
    REQUIRE((*static_cast<RealStorage *>(host.get()))[5] == R(36));
    StoragePtr back = host->gpu();
    REQUIRE(back->device == DeviceTag::GPU);
    REQUIRE((*static_cast<RealStorage *>(back.get()))[4] == R(35));
    static_cast<RealStorage *>(back.get())->write(4U, R(-1));
    REQUIRE((*static_cast<RealStorage *>(back.get()))[4] == R(-1));
    REQUIRE_THROWS_AS((*static_cast<RealStorage *>(back.get()))[6], std::invalid_argument);
    REQUIRE_THROWS_AS(a + Tensor::transpose(a), std::invalid_argument);
}

// --------------------------------------------------------------------------------------------------------------------
// QuantizedKVCache
// --------------------------------------------------------------------------------------------------------------------

TEST_CASE(test_quantized_cache_known_answers, true)
{
    // write_row / read_row answers recorded from the reference's own coder, padded with zeros to d = 32
    const std::vector<real1> vals = { -10, -3, -2.999f, -1e-4f, 0, .1874f, .1876f, 2.6249f, 2.625f, 2.99f, 3, 10 };
    struct Kat {
        int bits;
        std::vector<uint32_t> words; // the words that hold the twelve codes
    };
    for (const Kat &k : { Kat{ 2, { 0x00ffea40u } }, Kat{ 3, { 0x3ff24600u, 0x0000003fu } }, Kat{ 4, { 0xe8887000u, 0x0000ffffu } } }) {
        QuantizedKVCache qc;
        qc.allocate(4U, 32U, k.bits);
        qc.block_scale = ONE_R1;
        std::vector<real1> row(32, -10.0f); // padding codes are 0, so the known words are not disturbed
        std::copy(vals.begin(), vals.end(), row.begin());
        qc.write_row(0U, row.data());
        qc.sync_packed();
        for (size_t w = 0; w < k.words.size(); ++w) {
            REQUIRE((uint32_t)qc.packed[w] == k.words[w]);
        }
        // the whole row against the CPU checker, words and dequantised values
        std::vector<int32_t> want_words((size_t)wo_words_per_row(32, k.bits), 0);
        wo_uniform_write_row(want_words.data(), 0U, row.data(), 32, k.bits, 1.0f);
        REQUIRE(qc.packed.size() == want_words.size());
        REQUIRE(std::memcmp(qc.packed.data(), want_words.data(), want_words.size() * sizeof(int32_t)) == 0);
        std::vector<real1> got(32), want(32);
        qc.read_row(0U, got.data());
        wo_uniform_read_row(want_words.data(), 0U, want.data(), 32, k.bits, 1.0f);
        REQUIRE(got == want);
        REQUIRE_THROWS_AS(qc.write_row(3U, row.data()), std::domain_error); // append-only
    }
    {
        QuantizedKVCache qc;
        qc.allocate(2U, 32U, 4);
        qc.block_scale = 0.731f;
        std::vector<real1> row(32, -10.0f);
        const real1 in[4] = { 0.5f, -1.2f, 2.0f, -0.05f };
        std::copy(in, in + 4, row.begin());
        qc.write_row(0U, row.data());
        qc.sync_packed();
        REQUIRE(((uint32_t)qc.packed[0] & 0xffffu) == 0x7f39u);
        std::vector<real1> got(32);
        qc.read_row(0U, got.data());
        REQUIRE(got[0] == 0.41118741f);
        REQUIRE(got[1] == -1.23356247f);
        REQUIRE(got[2] == 2.05593753f);
        REQUIRE(got[3] == -0.13706255f);
    }
}

// --------------------------------------------------------------------------------------------------------------------
// MultiHeadAttention
// --------------------------------------------------------------------------------------------------------------------

struct HostLinear {
    std::vector<real1> w, b; // w column-major (in, out)
    tcapint in, out;
};

HostLinear install(const LinearPtr &l, uint32_t seed)
{
    HostLinear h;
    h.in = l->in_features;
    h.out = l->out_features;
    h.w = gaussian((size_t)h.in * h.out, seed, 1.0f / std::sqrt((real1)h.in));
    h.b = gaussian(h.out, seed + 1U, 0.1f);
    l->weight = std::make_shared<Parameter>(h.w, std::vector<tcapint>{ h.in, h.out }, true, TEST_DTAG);
    if (l->bias) {
        l->bias = std::make_shared<Parameter>(h.b, std::vector<tcapint>{ 1U, h.out }, true, TEST_DTAG);
    }
    return h;
}

// y[r, o] = sum_i x[r, i] w[i, o] + b[o] in double; x is column-major (rows, in)
std::vector<double> host_linear(const HostLinear &l, const std::vector<double> &x, size_t rows)
{
    std::vector<double> y(rows * l.out);
    for (size_t r = 0; r < rows; ++r) {
        for (tcapint o = 0; o < l.out; ++o) {
            double acc = l.b[o];
            for (tcapint i = 0; i < l.in; ++i) {
                acc += x[r + rows * i] * (double)l.w[i + (size_t)l.in * o];
            }
            y[r + rows * o] = acc;
        }
    }
    return y;
}

// Dense float64 attention over given K/V rows (already what the cache holds), as MultiHeadAttention::forward
// defines it: element (b, t, h, j) of a (B, T, H, hd) column-major tensor is at b + B*(t + T*(h + H*j)).
struct AttnCheck {
    tcapint B, H, Hkv, hd;
    bool blocked;
    // kv(b, kvh, tok, j): cached row value
    std::function<double(tcapint, tcapint, tcapint, tcapint)> kf, vf;
};

std::vector<double> host_attention(const AttnCheck &g, const std::vector<double> &Q, tcapint T, tcapint before)
{
    std::vector<double> out((size_t)g.B * T * g.H * g.hd, 0.0);
    const tcapint groups = g.H / g.Hkv;
    for (tcapint b = 0; b < g.B; ++b) {
        for (tcapint t = 0; t < T; ++t) {
            for (tcapint h = 0; h < g.H; ++h) {
                const tcapint kvh = g.blocked ? h / groups : h % g.Hkv;
                const tcapint n = before + t + 1U;
                std::vector<double> s(n);
                double mx = -1e300;
                for (tcapint tok = 0; tok < n; ++tok) {
                    double acc = 0.0;
                    for (tcapint j = 0; j < g.hd; ++j) {
                        acc += Q[b + (size_t)g.B * (t + (size_t)T * (h + (size_t)g.H * j))] * g.kf(b, kvh, tok, j);
                    }
                    s[tok] = acc / std::sqrt((double)g.hd);
                    mx = std::max(mx, s[tok]);
                }
                double sum = 0.0;
                for (double &v : s) {
                    v = std::exp(v - mx);
                    sum += v;
                }
                for (tcapint j = 0; j < g.hd; ++j) {
                    double acc = 0.0;
                    for (tcapint tok = 0; tok < n; ++tok) {
                        acc += s[tok] * g.vf(b, kvh, tok, j);
                    }
                    out[b + (size_t)g.B * (t + (size_t)T * (h + (size_t)g.H * j))] = acc / sum;
                }
            }
        }
    }
    return out;
}

// y = x.R over the last (slowest) dimension of a column-major (rows, hd) array
std::vector<double> host_rotate(const std::vector<double> &x, size_t rows, tcapint hd, const std::vector<real1> &Rm)
{
    std::vector<double> y(rows * hd);
    for (size_t r = 0; r < rows; ++r) {
        for (tcapint j = 0; j < hd; ++j) {
            double acc = 0.0;
            for (tcapint i = 0; i < hd; ++i) {
                acc += x[r + rows * i] * (double)Rm[i + (size_t)hd * j];
            }
            y[r + rows * j] = acc;
        }
    }
    return y;
}

std::vector<double> to_double(const std::vector<real1> &v) { return std::vector<double>(v.begin(), v.end()); }

// RoPE on a (B, T, H, hd) column-major array in double, positions pos0 + t, with the module's own tables
std::vector<double> host_rope(const std::vector<double> &x, tcapint B, tcapint T, tcapint H, tcapint hd, const RoPE &rope,
    tcapint pos0)
{
    const std::vector<real1> ct = rope.cos_table->to_vector(), st = rope.sin_table->to_vector();
    std::vector<double> y(x.size());
    const tcapint half = hd / 2U, L = rope.max_seq_len;
    for (tcapint b = 0; b < B; ++b) {
        for (tcapint t = 0; t < T; ++t) {
            for (tcapint h = 0; h < H; ++h) {
                for (tcapint j = 0; j < hd; ++j) {
                    auto at = [&](tcapint jj) { return x[b + (size_t)B * (t + (size_t)T * (h + (size_t)H * jj))]; };
                    const double partner = j < half ? -at(j + half) : at(j - half);
                    const size_t ti = (pos0 + t) + (size_t)j * L;
                    y[b + (size_t)B * (t + (size_t)T * (h + (size_t)H * j))] = at(j) * (double)ct[ti] + partner * (double)st[ti];
                }
            }
        }
    }
    return y;
}

TEST_CASE(test_rope_matches_checker, true)
{
    // tables and forward pass against the CPU checker's restatement of src/modules/rope.cpp, bit for bit
    const tcapint B = 2U, H = 3U, T = 5U, hd = 32U, L = 24U;
    RoPE rope(hd, L, 10000.0f, TEST_DTAG);
    std::vector<real1> ct((size_t)L * hd), st((size_t)L * hd);
    wo_rope_tables(hd, L, 10000.0f, ct.data(), st.data());
    REQUIRE(rope.cos_table->to_vector() == ct);
    REQUIRE(rope.sin_table->to_vector() == st);
    const std::vector<real1> xc = gaussian((size_t)B * H * T * hd, 8U); // C order [B][H][T][hd] for the checker
    std::vector<real1> xcm(xc.size());                                   // column-major for the tensor
    for (tcapint b = 0; b < B; ++b)
        for (tcapint h = 0; h < H; ++h)
            for (tcapint t = 0; t < T; ++t)
                for (tcapint j = 0; j < hd; ++j)
                    xcm[b + (size_t)B * (h + (size_t)H * (t + (size_t)T * j))] = xc[(((size_t)b * H + h) * T + t) * hd + j];
    TensorPtr x = std::make_shared<Tensor>(xcm, std::vector<tcapint>{ B, H, T, hd }, false, TEST_DTAG);
    for (const tcapint pos0 : { 0U, 7U }) {
        std::vector<real1> want(xc.size());
        wo_rope_forward(xc.data(), B, H, T, hd, ct.data(), st.data(), L, pos0, want.data());
        const std::vector<real1> got = rope.forward(x, pos0)->to_vector();
        bool same = true;
        for (tcapint b = 0; b < B && same; ++b)
            for (tcapint h = 0; h < H && same; ++h)
                for (tcapint t = 0; t < T && same; ++t)
                    for (tcapint j = 0; j < hd && same; ++j)
                        same = got[b + (size_t)B * (h + (size_t)H * (t + (size_t)T * j))] == want[(((size_t)b * H + h) * T + t) * hd + j];
        REQUIRE(same);
    }
    REQUIRE(rope.forward(x)->to_vector() == rope.forward(x, 0U)->to_vector());
    REQUIRE_THROWS_AS(rope.forward(x, L - T + 1U), std::out_of_range);
    REQUIRE_THROWS_AS(std::make_shared<RoPE>(31U, L), std::invalid_argument);
}

void run_attention_case(KVCoder coder, int bits, bool blocked, uint32_t seed, bool with_rope = false)
{
    const tcapint B = 2U, dm = 96U, H = 4U, Hkv = 2U, hd = 64U;
    RoPEPtr rope = with_rope ? std::make_shared<RoPE>(hd, 40U, 10000.0f, TEST_DTAG) : nullptr;
    MultiHeadAttention mha(dm, H, Hkv, hd, TEST_DTAG, rope, ZERO_R1, -1, true, bits);
    mha.kv_coder = coder;
    mha.gqa_blocked = blocked;
    mha.rotation_seed = seed;
    if (coder == KV_LLOYDMAX) {
        mha.k_bits = 3;
        mha.k_sign = true;
    }
    mha.set_max_kv_seq_len(40U);
    const HostLinear wq = install(mha.W_q, seed + 10U), wk = install(mha.W_k, seed + 20U);
    const HostLinear wv = install(mha.W_v, seed + 30U), wo = install(mha.W_o, seed + 40U);
    (void)wk;
    (void)wv;

    tcapint before = 0U;
    // prefill, two decode steps, a chunk, a long chunk on the dense path, a long chunk in groups through the fused kernel
    const std::pair<tcapint, MultiHeadAttention::PrefillPath> calls[] = { { 7U, MultiHeadAttention::PREFILL_AUTO },
        { 1U, MultiHeadAttention::PREFILL_AUTO }, { 1U, MultiHeadAttention::PREFILL_AUTO },
        { 3U, MultiHeadAttention::PREFILL_AUTO }, { 12U, MultiHeadAttention::PREFILL_DENSE },
        { 9U, MultiHeadAttention::PREFILL_FUSED } };
    for (const auto &call : calls) {
        const tcapint T = call.first;
        mha.prefill_path = call.second;
        const std::vector<real1> xv = gaussian((size_t)B * T * dm, seed + 100U + before);
        TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, dm }, false, TEST_DTAG);
        TensorPtr y = mha.forward(x);
        REQUIRE(y->shape == (std::vector<tcapint>{ B, T, dm }));
        REQUIRE(mha.cache_len == before + T);
        REQUIRE(mha.max_seq_len == 40U); // the reference overwrites this at the first call; here it sticks
        REQUIRE(mha.k_rotation.size() == (size_t)hd * hd);

        // check: float64 attention over the rows the device cache actually holds (rotated basis)
        const size_t rows = (size_t)B * T;
        std::vector<double> Qd = host_linear(wq, to_double(xv), rows); // (B, T, H*hd) = (B, T, H, hd)
        if (with_rope) {
            Qd = host_rope(Qd, B, T, H, hd, *rope, before); // the query sits at positions before .. before + T - 1
        }
        Qd = host_rotate(Qd, rows * H, hd, mha.k_rotation);
        const tcapint cap = mha.max_seq_len;
        std::vector<real1> krows((size_t)B * Hkv * (before + T) * hd), vrows(krows.size());
        for (tcapint p = 0; p < B * Hkv; ++p) {
            for (tcapint tok = 0; tok < before + T; ++tok) {
                mha.k_qcache.read_row(p * cap + tok, &krows[((size_t)p * (before + T) + tok) * hd]);
                mha.v_qcache.read_row(p * cap + tok, &vrows[((size_t)p * (before + T) + tok) * hd]);
            }
        }
        const tcapint n_tok = before + T;
        AttnCheck g{ B, H, Hkv, hd, blocked,
            [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return (double)krows[(((size_t)(b * Hkv + kvh)) * n_tok + tok) * hd + j]; },
            [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return (double)vrows[(((size_t)(b * Hkv + kvh)) * n_tok + tok) * hd + j]; } };
        std::vector<double> att = host_attention(g, Qd, T, before);
        att = host_rotate(att, rows * H, hd, mha.v_rotation_trans);
        const std::vector<double> want = host_linear(wo, att, rows);
        double worst = 0.0;
        const bool ok = attn_close(y->to_vector(), want, &worst);
        if (!ok) {
            std::printf("    coder %d bits %d T %u before %u: worst abs err %.3e\n", (int)coder, bits, T, before, worst);
        }
        REQUIRE(ok);
        before += T;
    }

    // the cached rows are the coder's image of the rotated projections: compare one pair with the CPU checker
    if (coder == KV_UNIFORM) {
        mha.k_qcache.sync_packed();
        REQUIRE(mha.k_qcache.packed.size() == (size_t)B * Hkv * before * (size_t)wo_words_per_row((int)hd, bits));
        REQUIRE(mha.k_qcache.block_scale > 0.0f);
        REQUIRE(mha.k_qcache.outer == B * Hkv * before);
    }

    // lifecycle (include/modules/multihead_attention.hpp:138-149)
    const std::vector<real1> big = gaussian((size_t)B * 30U * dm, seed + 7U);
    REQUIRE_THROWS_AS(mha.forward(std::make_shared<Tensor>(big, std::vector<tcapint>{ B, 30U, dm }, false, TEST_DTAG)),
        std::out_of_range);
    REQUIRE_THROWS_AS(mha.forward(std::make_shared<Tensor>(gaussian(3U * dm, 1U), std::vector<tcapint>{ 3U, 1U, dm }, false, TEST_DTAG)),
        std::invalid_argument);
    mha.reset_cache();
    REQUIRE(mha.cache_len == 0U);
    REQUIRE(mha.max_seq_len == 0U);
    REQUIRE(mha.k_rotation.empty());
    REQUIRE(mha.k_qcache.d == 0U);
    TensorPtr y = mha.forward(std::make_shared<Tensor>(gaussian(3U * dm, 1U), std::vector<tcapint>{ 3U, 1U, dm }, false, TEST_DTAG));
    REQUIRE(y->shape == (std::vector<tcapint>{ 3U, 1U, dm }));
    REQUIRE(mha.max_seq_len == (with_rope ? 40U : 2048U)); // the reference's default capacity (cpp:173)
}

TEST_CASE(test_prefill_path_estimate, true)
{
    // Llama-like shape, 3 + 4 bit rows: a few new tokens against long contexts stay on the packed cache, a long
    // prefill of one sequence is dequantised once; forcing either path is covered by run_attention_case
    MultiHeadAttention mha(4096U, 32U, 8U, 128U, TEST_DTAG, nullptr, ZERO_R1, -1, true, 4);
    mha.kv_coder = KV_LLOYDMAX;
    mha.k_bits = 3;
    REQUIRE(!mha.dense_is_cheaper(64U, 4U, 8192U));
    REQUIRE(!mha.dense_is_cheaper(64U, 64U, 8192U));
    REQUIRE(!mha.dense_is_cheaper(1U, 8U, 300U));
    REQUIRE(mha.dense_is_cheaper(1U, 4096U, 4096U));
    REQUIRE(mha.dense_is_cheaper(8U, 2048U, 2048U));
}

TEST_CASE(test_attention_uniform_4bit, true) { run_attention_case(KV_UNIFORM, 4, false, 1234U); }
TEST_CASE(test_attention_uniform_3bit_blocked_gqa, true) { run_attention_case(KV_UNIFORM, 3, true, 99U); }
TEST_CASE(test_attention_lloydmax, true) { run_attention_case(KV_LLOYDMAX, 4, false, 4321U); }
TEST_CASE(test_attention_with_rope, true) { run_attention_case(KV_LLOYDMAX, 4, false, 777U, true); }
// 8-bit codes (any kv_quant_bits the reference takes): no matrix-core tiles for such fields, every call goes through
// the generic kernel position by position, or densely
TEST_CASE(test_attention_uniform_8bit, true) { run_attention_case(KV_UNIFORM, 8, true, 31U); }

TEST_CASE(test_attention_uniform_codes_follow_reference_coder, true)
{
    // one call, B = 1, H = Hkv = 1, identity projections: the cached words must be exactly what the reference's
    // write_row makes of x.R (rotation in ascending order, sequential block scale), i.e. the CPU checker's words
    const tcapint T = 9U, hd = 64U;
    MultiHeadAttention mha(hd, 1U, 1U, hd, TEST_DTAG, nullptr, ZERO_R1, -1, true, 4, false);
    mha.rotation_seed = 5U;
    std::vector<real1> eye((size_t)hd * hd, 0.0f);
    for (tcapint i = 0; i < hd; ++i) {
        eye[i + (size_t)hd * i] = 1.0f;
    }
    for (const LinearPtr &l : { mha.W_q, mha.W_k, mha.W_v, mha.W_o }) {
        l->weight = std::make_shared<Parameter>(eye, std::vector<tcapint>{ hd, hd }, true, TEST_DTAG);
    }
    const std::vector<real1> xv = gaussian((size_t)T * hd, 77U); // (1, T, hd) column-major: row t is x[t + T*i]
    mha.forward(std::make_shared<Tensor>(xv, std::vector<tcapint>{ 1U, T, hd }, false, TEST_DTAG));
    std::vector<real1> rows((size_t)T * hd), rot((size_t)T * hd);
    for (tcapint t = 0; t < T; ++t) {
        for (tcapint i = 0; i < hd; ++i) {
            rows[(size_t)t * hd + i] = xv[t + (size_t)T * i];
        }
    }
    for (int which = 0; which < 2; ++which) {
        QuantizedKVCache &qc = which ? mha.v_qcache : mha.k_qcache;
        wo_apply_rotation(rows.data(), T, (int)hd, (which ? mha.v_rotation : mha.k_rotation).data(), rot.data());
        // the module sums squares in the memory order of its (B, T, heads, hd) tensor: i-major, t-minor
        std::vector<real1> flat((size_t)T * hd);
        for (tcapint t = 0; t < T; ++t) {
            for (tcapint i = 0; i < hd; ++i) {
                flat[t + (size_t)T * i] = rot[(size_t)t * hd + i];
            }
        }
        const real1 scale = wo_block_scale(flat.data(), flat.size());
        REQUIRE(std::fabs(qc.block_scale - scale) <= 2e-7f * scale);
        std::vector<int32_t> want((size_t)T * wo_words_per_row((int)hd, 4), 0);
        wo_uniform_write_rows(want.data(), rot.data(), T, (int)hd, 4, qc.block_scale);
        qc.sync_packed();
        REQUIRE(qc.packed.size() == want.size());
        REQUIRE(std::memcmp(qc.packed.data(), want.data(), want.size() * sizeof(int32_t)) == 0);
    }
}

TEST_CASE(test_attention_dense_path_matches_quantized_at_fine_steps, true)
{
    // float cache (kv_quant_bits = 0) and no cache: the reference's own sequence of dense ops, on the device.
    // Incremental calls must equal one call over the whole sequence, and both must equal float64 attention.
    const tcapint B = 2U, dm = 48U, H = 4U, Hkv = 2U, hd = 16U, T = 6U;
    MultiHeadAttention cached(dm, H, Hkv, hd, TEST_DTAG, nullptr, ZERO_R1, -1, true, 0);
    MultiHeadAttention oneshot(dm, H, Hkv, hd, TEST_DTAG, nullptr, ZERO_R1, -1, false, 0);
    cached.set_max_kv_seq_len(16U);
    const HostLinear wq = install(cached.W_q, 1U), wk = install(cached.W_k, 2U), wv = install(cached.W_v, 3U),
                     wo = install(cached.W_o, 4U);
    install(oneshot.W_q, 1U);
    install(oneshot.W_k, 2U);
    install(oneshot.W_v, 3U);
    install(oneshot.W_o, 4U);
    const std::vector<real1> xv = gaussian((size_t)B * T * dm, 55U);
    TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, dm }, false, TEST_DTAG);
    const std::vector<real1> whole = oneshot.forward(x)->to_vector();

    const size_t rows = (size_t)B * T;
    const std::vector<double> Qd = host_linear(wq, to_double(xv), rows), Kd = host_linear(wk, to_double(xv), rows),
                              Vd = host_linear(wv, to_double(xv), rows);
    AttnCheck g{ B, H, Hkv, hd, false,
        [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return Kd[b + (size_t)B * (tok + (size_t)T * (kvh + (size_t)Hkv * j))]; },
        [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return Vd[b + (size_t)B * (tok + (size_t)T * (kvh + (size_t)Hkv * j))]; } };
    const std::vector<double> want = host_linear(wo, host_attention(g, Qd, T, 0U), rows);
    REQUIRE(attn_close(whole, want));

    // prefill 4 tokens, then 2 single-token steps, against the matching slices of the one-shot result
    std::vector<real1> pieces(whole.size());
    tcapint done = 0U;
    for (const tcapint step : { 4U, 1U, 1U }) {
        TensorPtr xs = Tensor::contiguous(Tensor::slice(x, 1, done, step));
        const std::vector<real1> ys = cached.forward(xs)->to_vector(); // (B, step, dm)
        for (tcapint f = 0; f < dm; ++f) {
            for (tcapint t = 0; t < step; ++t) {
                for (tcapint b = 0; b < B; ++b) {
                    pieces[b + (size_t)B * ((done + t) + (size_t)T * f)] = ys[b + (size_t)B * (t + (size_t)step * f)];
                }
            }
        }
        done += step;
    }
    REQUIRE(attn_close(pieces, want));
    REQUIRE(cached.cache_len == T);
}


// ---- checkpoint streams (weed_amd/host/serialize.cpp).  The reference has no test or fixture of its streams; the
//      expected bytes below are assembled by hand from its writer code (serializer.hpp, storage.cpp:25-30,
//      parameter.cpp:16-31, linear.cpp:109-118, rope.cpp:100-106, multihead_attention.cpp:358-375). ----
struct Bytes {
    std::string b;
    Bytes &u8(uint8_t v)
    {
        b.push_back((char)v);
        return *this;
    }
    Bytes &u32(uint32_t v)
    {
        for (int i = 0; i < 4; ++i) {
            b.push_back((char)((v >> (8 * i)) & 0xff));
        }
        return *this;
    }
    Bytes &f32(float v)
    {
        uint32_t w;
        std::memcpy(&w, &v, 4);
        return u32(w);
    }
};

TEST_CASE(test_integer_storage_on_the_host, false)
{
    // symbol-table storage (include/storage/cpu_int_storage.hpp): fills, element access, stream bytes
    std::shared_ptr<CpuIntStorage> sp = std::make_shared<CpuIntStorage>(std::vector<symint>{ 7, -2, 40000 });
    CpuIntStorage &s = *sp;
    REQUIRE(s.dtype == DType::INT && s.stype == INT_CPU_DENSE && s.size == 3U);
    REQUIRE(s[1U] == -2);
    s.add(1U, 5);
    REQUIRE(s[1U] == 3);
    REQUIRE_THROWS_AS(s[3U], std::invalid_argument);
    REQUIRE_THROWS_AS(std::make_shared<CpuIntStorage>(0U), std::invalid_argument);
    std::ostringstream os;
    s.save(os);
    Bytes e;
    e.u32(5U).u32(0xffffffffU).u32(0xffffffffU).u32(3U); // INT_CPU_DENSE, 8-byte device id -1, 3 elements
    e.u32(7U).u32(3U).u32(40000U);
    REQUIRE(os.str() == e.b);
    std::istringstream is(e.b);
    std::shared_ptr<CpuIntStorage> r = std::dynamic_pointer_cast<CpuIntStorage>(Storage::load(is));
    REQUIRE(r && r->data == (std::vector<symint>{ 7, 3, 40000 }));
    s.FillOnes();
    REQUIRE(s.data == (std::vector<symint>{ 1, 1, 1 }));
    s.FillValue(-9);
    REQUIRE(s[2U] == -9);
    s.FillZeros();
    REQUIRE(s[0U] == 0);
}

TEST_CASE(test_integer_storage_on_the_device, true)
{
    // include/storage/gpu_int_storage.hpp: allocation, fills, blocking transfers both ways, stream round trip
    std::vector<symint> ids(1000);
    for (size_t i = 0; i < ids.size(); ++i) {
        ids[i] = (symint)(i * 37 % 501) - 250;
    }
    std::shared_ptr<GpuIntStorage> g = std::make_shared<GpuIntStorage>(ids);
    REQUIRE(g->device == DeviceTag::GPU && g->dtype == DType::INT && g->stype == INT_GPU_DENSE);
    REQUIRE((*g)[0U] == ids[0] && (*g)[999U] == ids[999]);
    REQUIRE_THROWS_AS((*g)[1000U], std::invalid_argument);
    REQUIRE_THROWS_AS(g->write(0U, 1), std::domain_error); // as the reference: no element writes on a device
    std::shared_ptr<CpuIntStorage> back = std::dynamic_pointer_cast<CpuIntStorage>(g->cpu());
    REQUIRE(back && back->data == ids);
    std::shared_ptr<GpuIntStorage> up = std::dynamic_pointer_cast<GpuIntStorage>(back->gpu());
    REQUIRE(up && (*up)[123U] == ids[123]);
    std::ostringstream os;
    g->save(os);
    std::istringstream is(os.str());
    std::shared_ptr<GpuIntStorage> r = std::dynamic_pointer_cast<GpuIntStorage>(Storage::load(is));
    REQUIRE(r && std::dynamic_pointer_cast<CpuIntStorage>(r->cpu())->data == ids);
    GpuIntStorage z(64U);
    z.FillOnes();
    REQUIRE(z[63U] == 1);
    z.FillValue(-5);
    REQUIRE(z[0U] == -5 && z[63U] == -5);
    z.FillZeros();
    REQUIRE(z[31U] == 0);
}

TEST_CASE(test_checkpoint_linear_known_bytes, false)
{
    // host-side storage: serialization needs no device
    Linear l(2U, 3U, true, false, DType::REAL, DeviceTag::CPU);
    const std::vector<real1> w{ 1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f }, b{ 0.5f, -1.0f, 2.0f };
    for (tcapint i = 0; i < 6U; ++i) {
        std::dynamic_pointer_cast<RealStorage>(l.weight->storage)->write(i, w[i]);
    }
    for (tcapint i = 0; i < 3U; ++i) {
        std::dynamic_pointer_cast<RealStorage>(l.bias->storage)->write(i, b[i]);
    }
    std::ostringstream os;
    l.save(os);

    Bytes e;
    e.u32(2U);                                  // LINEAR_T
    e.u32(2U).u32(3U);                          // in_features, out_features
    e.u32(0xffffffffU).u32(0U).u32(2U);         // weight: device id -1, offset 0, rank 2
    e.u32(2U).u32(1U).u32(3U).u32(2U);          // (shape, stride) of the column-major 2 x 3 matrix
    e.u32(1U).u32(0xffffffffU).u32(0xffffffffU).u32(6U); // storage: REAL_CPU_DENSE, 8-byte device id -1, 6 elements
    for (float v : w) {
        e.f32(v);
    }
    e.u8(1U);                                   // has bias
    e.u32(0xffffffffU).u32(0U).u32(2U);         // bias: device id -1, offset 0, rank 2
    e.u32(1U).u32(0U).u32(3U).u32(1U);          // (1, 3): the size-1 dimension has stride 0
    e.u32(1U).u32(0xffffffffU).u32(0xffffffffU).u32(3U);
    for (float v : b) {
        e.f32(v);
    }
    REQUIRE(os.str() == e.b);

    // reading the hand-assembled bytes gives the module back; the upper half of the 8-byte device id is ignored
    std::string junk = e.b;
    junk[4 * 11 + 4] = (char)0x5a; // first byte of the undefined upper half in the weight's storage record
    for (const std::string &src : { e.b, junk }) {
        std::istringstream is(src);
        LinearPtr r = std::dynamic_pointer_cast<Linear>(Module::load(is));
        REQUIRE(r && r->in_features == 2U && r->out_features == 3U && r->bias);
        if (r && r->bias) {
            REQUIRE(r->weight->shape == (std::vector<tcapint>{ 2U, 3U }) && r->weight->stride == (std::vector<tcapint>{ 1U, 2U }));
            REQUIRE(r->bias->shape == (std::vector<tcapint>{ 1U, 3U }) && r->bias->stride == (std::vector<tcapint>{ 0U, 1U }));
            REQUIRE(r->weight->to_vector() == w && r->bias->to_vector() == b);
            REQUIRE(r->weight->storage->device == DeviceTag::CPU);
        }
        REQUIRE(is.peek() == std::char_traits<char>::eof()); // the record was consumed exactly
    }

    // error paths: truncated stream, foreign module tag, foreign storage tag
    {
        std::istringstream is(e.b.substr(0, e.b.size() - 3));
        REQUIRE_THROWS_AS(Module::load(is), std::runtime_error);
    }
    {
        std::istringstream is(Bytes().u32(8U).b); // EMBEDDING_T in the reference: not a module of this path
        REQUIRE_THROWS_AS(Module::load(is), std::domain_error);
    }
    {
        std::string bad = e.b;
        bad[4 * 10] = 3; // COMPLEX_CPU_DENSE
        std::istringstream is(bad);
        REQUIRE_THROWS_AS(Module::load(is), std::domain_error);
    }
}

TEST_CASE(test_checkpoint_attention_header_bytes, false)
{
    // the fixed-size part of an attention record: tag, mask value, four sizes, cache flag, bit width
    MultiHeadAttention m(8U, 2U, 1U, 4U, DeviceTag::CPU, nullptr, -5.0f, -1, true, 3, false);
    std::ostringstream os;
    m.save(os);
    Bytes e;
    e.u32(17U).f32(-5.0f).u32(8U).u32(2U).u32(1U).u32(4U).u8(1U).u32(3U);
    REQUIRE(os.str().size() > e.b.size() && os.str().compare(0, e.b.size(), e.b) == 0);
    // ... four bias-free projections follow: W_q 8x8, W_k 8x4, W_v 8x4, W_o 8x8, then "no RoPE"
    const size_t lin = 4U * 3U + 4U * 7U + 4U * 4U + 1U; // tag + sizes, parameter header (rank 2), storage header, bias flag
    const size_t want = e.b.size() + 4U * lin + 4U * (64U + 32U + 32U + 64U) + 1U;
    REQUIRE(os.str().size() == want);
    REQUIRE(os.str().back() == '\0');
    // a RoPE record: tag 31, head_dim, max_seq_len, base
    std::ostringstream ro;
    RoPE(4U, 16U, 10000.0f, DeviceTag::CPU).save(ro);
    REQUIRE(ro.str() == Bytes().u32(31U).u32(4U).u32(16U).f32(10000.0f).b);
}

TEST_CASE(test_checkpoint_attention_round_trip, true)
{
    // save -> load -> the same outputs, prefill and decode, with RoPE and the Lloyd-Max coder; the quantizer record
    // carries the coder settings and the rotations, so the reloaded module also produces the same cache words
    const tcapint B = 2U, dm = 64U, H = 4U, Hkv = 2U, hd = 32U;
    RoPEPtr rope = std::make_shared<RoPE>(hd, 32U, 10000.0f, TEST_DTAG);
    MultiHeadAttention a(dm, H, Hkv, hd, TEST_DTAG, rope, ZERO_R1, -1, true, 4);
    a.kv_coder = KV_LLOYDMAX;
    a.k_bits = 3;
    a.v_bits = 4;
    a.rotation_seed = 4242U;
    a.set_max_kv_seq_len(32U);
    const std::vector<real1> x0 = gaussian((size_t)B * 5U * dm, 11U), x1 = gaussian((size_t)B * dm, 12U);
    TensorPtr t0 = std::make_shared<Tensor>(x0, std::vector<tcapint>{ B, 5U, dm }, false, TEST_DTAG);
    TensorPtr t1 = std::make_shared<Tensor>(x1, std::vector<tcapint>{ B, 1U, dm }, false, TEST_DTAG);
    const std::vector<real1> y0 = a.forward(t0)->to_vector(), y1 = a.forward(t1)->to_vector();

    std::stringstream ss;
    a.save(ss);
    a.save_quantizer(ss);
    MultiHeadAttentionPtr b = std::dynamic_pointer_cast<MultiHeadAttention>(Module::load(ss));
    REQUIRE((bool)b);
    if (!b) {
        return;
    }
    b->load_quantizer(ss);
    REQUIRE(ss.peek() == std::char_traits<char>::eof());
    REQUIRE(b->d_model == a.d_model && b->num_heads == a.num_heads && b->num_kv_heads == a.num_kv_heads &&
        b->head_dim == a.head_dim && b->kv_quant_bits == a.kv_quant_bits && b->use_kv_cache == a.use_kv_cache &&
        b->mask_val == a.mask_val);
    REQUIRE(b->rope && b->rope->head_dim == hd && b->rope->max_seq_len == 32U && b->rope->base == 10000.0f);
    REQUIRE(b->kv_coder == KV_LLOYDMAX && b->k_bits == 3 && b->v_bits == 4 && b->rotation_seed == 4242U &&
        b->max_seq_len == 32U);
    REQUIRE(b->k_rotation == a.k_rotation && b->v_rotation == a.v_rotation && b->k_rotation.size() == (size_t)hd * hd);
    REQUIRE(b->parameters().size() == a.parameters().size());
    for (size_t i = 0; i < a.parameters().size() && i < b->parameters().size(); ++i) {
        REQUIRE(b->parameters()[i]->to_vector() == a.parameters()[i]->to_vector());
        REQUIRE(b->parameters()[i]->storage->device == DeviceTag::GPU);
    }
    // bit-identical replay: same weights, same rotations, same kernels
    REQUIRE(b->forward(t0)->to_vector() == y0);
    REQUIRE(b->forward(t1)->to_vector() == y1);
    // a record that is not a quantizer record is refused, and so is loading one into a cache that holds tokens
    std::stringstream again;
    a.save_quantizer(again);
    REQUIRE_THROWS_AS(b->load_quantizer(again), std::logic_error);
    std::istringstream wrong(std::string(64, 'x'));
    b->reset_cache();
    REQUIRE_THROWS_AS(b->load_quantizer(wrong), std::runtime_error);
}

// --------------------------------------------------------------------------------------------------------------------
// norms, activations, SwiGLU and the two modules that call the attention module
// --------------------------------------------------------------------------------------------------------------------

// float64 versions of the pieces (column-major (rows, n) arrays: element (r, j) at r + rows * j)
std::vector<double> host_rms_norm(const std::vector<double> &x, size_t rows, tcapint n, const std::vector<real1> &w)
{
    std::vector<double> y(x.size());
    for (size_t r = 0; r < rows; ++r) {
        double sq = 0.0;
        for (tcapint j = 0; j < n; ++j) {
            sq += x[r + rows * j] * x[r + rows * j];
        }
        const double root = std::sqrt(sq / n + (double)FP_NORM_EPSILON);
        for (tcapint j = 0; j < n; ++j) {
            y[r + rows * j] = x[r + rows * j] / root * (double)w[j];
        }
    }
    return y;
}
std::vector<double> host_layer_norm(const std::vector<double> &x, size_t rows, tcapint n, const std::vector<real1> &g,
    const std::vector<real1> &b, double eps)
{
    std::vector<double> y(x.size());
    for (size_t r = 0; r < rows; ++r) {
        double mu = 0.0, var = 0.0;
        for (tcapint j = 0; j < n; ++j) {
            mu += x[r + rows * j];
        }
        mu /= n;
        for (tcapint j = 0; j < n; ++j) {
            var += (x[r + rows * j] - mu) * (x[r + rows * j] - mu);
        }
        const double root = std::sqrt(var / n + eps);
        for (tcapint j = 0; j < n; ++j) {
            y[r + rows * j] = (x[r + rows * j] - mu) / root * (double)g[j] + (double)b[j];
        }
    }
    return y;
}
double host_gelu(double v) { return 0.5 * v * (1.0 + std::tanh(0.7978845608028654 * (v + 0.044715 * v * v * v))); }
std::vector<double> plus(const std::vector<double> &a, const std::vector<double> &b)
{
    std::vector<double> y(a.size());
    for (size_t i = 0; i < a.size(); ++i) {
        y[i] = a[i] + b[i];
    }
    return y;
}
void set_param(const ParameterPtr &p, const std::vector<real1> &v, const std::vector<tcapint> &shape)
{
    Parameter fresh(v, shape, true, TEST_DTAG);
    p->storage = fresh.storage;
    p->shape = fresh.shape;
    p->stride = fresh.stride;
    p->offset = 0U;
}

// What MultiHeadAttention::forward returns for the (B, T, dm) input `xin` (float64) when `before` tokens were cached
// ahead of the call: float64 attention over the rows the device cache holds AFTER the call (as the kernels see them,
// rotated basis), so the coder's error is not part of the comparison.
std::vector<double> host_mha(MultiHeadAttention &mha, const HostLinear &wq, const HostLinear &wo, const std::vector<double> &xin,
    tcapint B, tcapint T, tcapint before)
{
    const tcapint H = (tcapint)mha.num_heads, Hkv = (tcapint)mha.num_kv_heads, hd = (tcapint)mha.head_dim;
    const size_t rows = (size_t)B * T;
    std::vector<double> Qd = host_linear(wq, xin, rows);
    if (mha.rope) {
        Qd = host_rope(Qd, B, T, H, hd, *mha.rope, before);
    }
    Qd = host_rotate(Qd, rows * H, hd, mha.k_rotation);
    const tcapint cap = mha.max_seq_len, n_tok = before + T;
    std::vector<real1> krows((size_t)B * Hkv * n_tok * hd), vrows(krows.size());
    for (tcapint p = 0; p < B * Hkv; ++p) {
        for (tcapint tok = 0; tok < n_tok; ++tok) {
            mha.k_qcache.read_row(p * cap + tok, &krows[((size_t)p * n_tok + tok) * hd]);
            mha.v_qcache.read_row(p * cap + tok, &vrows[((size_t)p * n_tok + tok) * hd]);
        }
    }
    AttnCheck g{ B, H, Hkv, hd, mha.gqa_blocked,
        [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return (double)krows[(((size_t)(b * Hkv + kvh)) * n_tok + tok) * hd + j]; },
        [&](tcapint b, tcapint kvh, tcapint tok, tcapint j) { return (double)vrows[(((size_t)(b * Hkv + kvh)) * n_tok + tok) * hd + j]; } };
    std::vector<double> att = host_attention(g, Qd, T, before);
    att = host_rotate(att, rows * H, hd, mha.v_rotation_trans);
    return host_linear(wo, att, rows);
}

TEST_CASE(test_activation_modules_reference_cases, true)
{
    // test/tests.cpp:230-244 (relu), 284-291 (sigmoid), 314-321 (tanh), forward values
    auto scalar = [](real1 v) { return std::make_shared<Tensor>(v, false, TEST_DTAG); };
    REQUIRE(get_real(Tensor::relu(scalar(R(2)))) == R(2));
    REQUIRE(get_real(Tensor::relu(scalar(R(-2)))) == R(0));
    REQUIRE(get_real(Tensor::sigmoid(scalar(R(0)))) == R(0.5));
    REQUIRE(get_real(Tensor::tanh(scalar(R(0)))) == R(0));
    // test/tests.cpp:111-120 with an axis: mean(1, 2, 3) = 2, and the axis stays with extent 1
    TensorPtr x = std::make_shared<Tensor>(std::vector<real1>{ R(1), R(4), R(2), R(5), R(3), R(6) }, std::vector<tcapint>{ 2, 3 },
        false, TEST_DTAG);
    TensorPtr m = Tensor::mean(x, 1);
    REQUIRE(m->shape == (std::vector<tcapint>{ 2U, 1U }));
    REQUIRE(m->to_vector() == (std::vector<real1>{ R(2), R(5) }));
    // modules against the CPU checker on a (B, T, features) tensor; relu bit for bit
    const std::vector<real1> v = gaussian(3U * 5U * 40U, 21U, 2.5f);
    TensorPtr t = std::make_shared<Tensor>(v, std::vector<tcapint>{ 3U, 5U, 40U }, false, TEST_DTAG);
    struct Act {
        std::shared_ptr<Module> m;
        int op;
        ModuleType tag;
    };
    for (const Act &a : { Act{ std::make_shared<ReLU>(), 0, RELU_T }, Act{ std::make_shared<Sigmoid>(), 1, SIGMOID_T },
             Act{ std::make_shared<Tanh>(), 2, TANH_T }, Act{ std::make_shared<GeLU>(), 3, GELU_T } }) {
        std::vector<real1> want(v.size());
        wo_unary(a.op, v.data(), v.size(), want.data());
        const std::vector<real1> got = a.m->forward(t)->to_vector();
        bool ok = got.size() == want.size();
        for (size_t i = 0; ok && i < got.size(); ++i) {
            ok = a.op == 0 ? got[i] == want[i] : std::fabs(got[i] - want[i]) <= 3e-7f + 2e-6f * std::fabs(want[i]);
        }
        REQUIRE(ok);
        // their stream is the tag alone (module.cpp:53-56, 87-98)
        std::ostringstream os;
        a.m->save(os);
        REQUIRE(os.str() == Bytes().u32((uint32_t)a.tag).b);
        std::istringstream is(os.str());
        std::shared_ptr<Module> r = Module::load(is);
        REQUIRE(r && r->mtype == a.tag);
    }
    REQUIRE_THROWS_AS(Tensor::relu(std::make_shared<Tensor>(v, std::vector<tcapint>{ 3U, 5U, 40U }, false, DeviceTag::CPU)),
        std::domain_error);
}

TEST_CASE(test_rms_norm_and_layer_norm_modules, true)
{
    // include/modules/rms_norm.hpp:34-38 and src/modules/layernorm.cpp:29-42 on (B, T, features) column-major tensors,
    // against the CPU checker (rows gathered for it) and float64
    const tcapint B = 3U, T = 4U, n = 96U;
    const std::vector<real1> v = gaussian((size_t)B * T * n, 31U, 3.0f);
    TensorPtr x = std::make_shared<Tensor>(v, std::vector<tcapint>{ B, T, n }, false, TEST_DTAG);
    const size_t rows = (size_t)B * T;
    std::vector<real1> dense(v.size()); // [row][n] for the checker
    for (size_t r = 0; r < rows; ++r) {
        for (tcapint j = 0; j < n; ++j) {
            dense[r * n + j] = v[r + rows * j];
        }
    }
    const std::vector<real1> w = gaussian(n, 32U, 0.3f), bt = gaussian(n, 33U);
    RMSNorm rms(n, -1, TEST_DTAG);
    REQUIRE(rms.weight->to_vector() == std::vector<real1>(n, ONE_R1)); // FillOnes (rms_norm.hpp:30)
    REQUIRE(rms.parameters().size() == 1U);
    set_param(rms.weight, w, { n });
    std::vector<real1> want(v.size());
    wo_rms_norm(dense.data(), rows, n, w.data(), wo_norm_epsilon(), want.data());
    std::vector<real1> got = rms.forward(x)->to_vector();
    std::vector<double> want64 = host_rms_norm(to_double(v), rows, n, w);
    bool ok = true, ok64 = true;
    for (size_t r = 0; r < rows; ++r) {
        for (tcapint j = 0; j < n; ++j) {
            ok = ok && std::fabs(got[r + rows * j] - want[r * n + j]) <= 2e-6f + 2e-6f * std::fabs(want[r * n + j]);
            ok64 = ok64 && std::fabs((double)got[r + rows * j] - want64[r + rows * j]) <= 2e-6 + 2e-6 * std::fabs(want64[r + rows * j]);
        }
    }
    REQUIRE(ok);
    REQUIRE(ok64);
    REQUIRE_THROWS_AS(RMSNorm(n + 1U, -1, TEST_DTAG).forward(x), std::invalid_argument);

    LayerNorm ln(n, TEST_DTAG);
    REQUIRE(ln.eps == FP_NORM_EPSILON && ln.gamma->shape == (std::vector<tcapint>{ 1U, 1U, n }));
    REQUIRE(ln.gamma->to_vector() == std::vector<real1>(n, ONE_R1) && ln.beta->to_vector() == std::vector<real1>(n, ZERO_R1));
    set_param(ln.gamma, w, { 1U, 1U, n });
    set_param(ln.beta, bt, { 1U, 1U, n });
    wo_layer_norm(dense.data(), rows, n, w.data(), bt.data(), ln.eps, want.data());
    got = ln.forward(x)->to_vector();
    want64 = host_layer_norm(to_double(v), rows, n, w, bt, (double)ln.eps);
    ok = ok64 = true;
    for (size_t r = 0; r < rows; ++r) {
        for (tcapint j = 0; j < n; ++j) {
            ok = ok && std::fabs(got[r + rows * j] - want[r * n + j]) <= 4e-6f + 4e-6f * std::fabs(want[r * n + j]);
            ok64 = ok64 && std::fabs((double)got[r + rows * j] - want64[r + rows * j]) <= 4e-6 + 4e-6 * std::fabs(want64[r + rows * j]);
        }
    }
    REQUIRE(ok);
    REQUIRE(ok64);
}

TEST_CASE(test_checkpoint_norm_and_swiglu_known_bytes, false)
{
    // hand-assembled from the reference's writers: rms_norm.hpp:39-44, layernorm.cpp:44-50, swiglu.cpp:18-25
    RMSNorm rms(3U, -1, DeviceTag::CPU);
    std::ostringstream os;
    rms.save(os);
    Bytes e;
    e.u32(30U).u32(0xffffffffU).u32(3U);            // RMS_NORM_T, axis -1, hidden_size
    e.u32(0xffffffffU).u32(0U).u32(1U).u32(3U).u32(1U); // weight: device id -1, offset 0, rank 1, (3, stride 1)
    e.u32(1U).u32(0xffffffffU).u32(0xffffffffU).u32(3U).f32(1.0f).f32(1.0f).f32(1.0f);
    REQUIRE(os.str() == e.b);
    {
        std::istringstream is(e.b);
        RMSNormPtr r = std::dynamic_pointer_cast<RMSNorm>(Module::load(is));
        REQUIRE(r && r->axis == -1 && r->hidden_size == 3U && r->weight->to_vector() == std::vector<real1>(3, 1.0f));
        REQUIRE(is.peek() == std::char_traits<char>::eof());
    }
    LayerNorm ln(2U, DeviceTag::CPU, 0.25f);
    std::dynamic_pointer_cast<RealStorage>(ln.beta->storage)->write(1U, -3.0f);
    std::ostringstream ol;
    ln.save(ol);
    Bytes l;
    l.u32(7U).u32(2U).f32(0.25f); // LAYERNORM_T, features, eps
    for (int which = 0; which < 2; ++which) {
        l.u32(0xffffffffU).u32(0U).u32(3U).u32(1U).u32(0U).u32(1U).u32(0U).u32(2U).u32(1U); // (1, 1, 2), strides (0, 0, 1)
        l.u32(1U).u32(0xffffffffU).u32(0xffffffffU).u32(2U);
        if (which == 0) {
            l.f32(1.0f).f32(1.0f);
        } else {
            l.f32(0.0f).f32(-3.0f);
        }
    }
    REQUIRE(ol.str() == l.b);
    {
        std::istringstream is(l.b);
        LayerNormPtr r = std::dynamic_pointer_cast<LayerNorm>(Module::load(is));
        REQUIRE(r && r->features == 2U && r->eps == 0.25f && r->beta->to_vector() == (std::vector<real1>{ 0.0f, -3.0f }));
        REQUIRE(r && r->gamma->shape == (std::vector<tcapint>{ 1U, 1U, 2U }));
    }
    // SwiGLU: tag, sizes, then three bias-free Linear records
    SwiGLU g(2U, 3U, DeviceTag::CPU);
    REQUIRE(g.parameters().size() == 3U);
    std::ostringstream og;
    g.save(og);
    const std::string head = Bytes().u32(32U).u32(2U).u32(3U).u32(2U).u32(2U).u32(3U).b; // ..., LINEAR_T, in 2, out 3
    REQUIRE(og.str().compare(0, head.size(), head) == 0);
    const size_t lin = 4U * 3U + 4U * 7U + 4U * 4U + 4U * 6U + 1U; // tag + sizes, parameter header, storage header, 6 floats, no bias
    REQUIRE(og.str().size() == 12U + 3U * lin);
    {
        std::istringstream is(og.str());
        SwiGLUPtr r = std::dynamic_pointer_cast<SwiGLU>(Module::load(is));
        REQUIRE(r && r->hidden_size == 2U && r->intermediate_size == 3U && r->parameters().size() == 3U);
        REQUIRE(r && r->down_proj->in_features == 3U && r->down_proj->out_features == 2U && !r->down_proj->bias);
        REQUIRE(r && r->gate_proj->weight->to_vector() == g.gate_proj->weight->to_vector());
    }
    // a record whose sub-module has the wrong type is refused
    {
        std::string bad = og.str();
        bad[12] = 31; // the gate projection's tag becomes ROPE_T
        std::istringstream is(bad);
        REQUIRE_THROWS_AS(Module::load(is), std::runtime_error);
    }
    REQUIRE_THROWS_AS(SwiGLU().forward(nullptr), std::domain_error);
}

TEST_CASE(test_transformer_encoder_layer_example_sizes, true)
{
    // The sizes of the reference's own example (examples/binary_addition_transformer.cpp:91-104: d_model 8, d_ff 16,
    // one head, 16 sequences of 6 tokens) through TransformerEncoderLayer::forward
    // (src/modules/transformer_encoder_layer.cpp:63-125), with the stock 4-bit cache, against float64:
    // x1 = x + attn(norm1(x)); out = x1 + ff2(gelu(ff1(norm2(x1)))).  A prefill and two decode steps.
    const tcapint B = 16U, dm = 8U, dff = 16U, H = 1U;
    TransformerEncoderLayer layer(dm, H, dff, TEST_DTAG, GELU_FN);
    REQUIRE(layer.parameters().size() == 8U + 2U + 2U + 2U + 2U);
    REQUIRE(layer.activation->mtype == GELU_T && layer.self_attn->head_dim == 8 && layer.self_attn->num_kv_heads == 1);
    layer.self_attn->rotation_seed = 17U;
    layer.set_max_kv_seq_len(16U);
    MultiHeadAttention &mha = *layer.self_attn;
    const HostLinear wq = install(mha.W_q, 101U), wk = install(mha.W_k, 102U), wv = install(mha.W_v, 103U), wo = install(mha.W_o, 104U);
    (void)wk;
    (void)wv;
    const HostLinear f1 = install(layer.ff1, 105U), f2 = install(layer.ff2, 106U);
    const std::vector<real1> g1 = gaussian(dm, 107U, 0.2f), b1 = gaussian(dm, 108U, 0.2f), g2 = gaussian(dm, 109U, 0.2f),
                             b2 = gaussian(dm, 110U, 0.2f);
    std::vector<real1> gamma1(dm), gamma2(dm);
    for (tcapint j = 0; j < dm; ++j) {
        gamma1[j] = 1.0f + g1[j];
        gamma2[j] = 1.0f + g2[j];
    }
    set_param(layer.norm1->gamma, gamma1, { 1U, 1U, dm });
    set_param(layer.norm1->beta, b1, { 1U, 1U, dm });
    set_param(layer.norm2->gamma, gamma2, { 1U, 1U, dm });
    set_param(layer.norm2->beta, b2, { 1U, 1U, dm });
    tcapint before = 0U;
    for (const tcapint T : { 6U, 1U, 1U }) {
        const std::vector<real1> xv = gaussian((size_t)B * T * dm, 200U + before);
        TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, dm }, false, TEST_DTAG);
        const std::vector<real1> got = layer.forward(x)->to_vector();
        REQUIRE(mha.cache_len == before + T && mha.max_seq_len == 16U);
        const size_t rows = (size_t)B * T;
        const std::vector<double> xd = to_double(xv);
        const std::vector<double> x1 = plus(xd, host_mha(mha, wq, wo, host_layer_norm(xd, rows, dm, gamma1, b1, FP_NORM_EPSILON), B, T, before));
        std::vector<double> ff = host_linear(f1, host_layer_norm(x1, rows, dm, gamma2, b2, FP_NORM_EPSILON), rows);
        for (double &v : ff) {
            v = host_gelu(v);
        }
        const std::vector<double> want = plus(x1, host_linear(f2, ff, rows));
        double worst = 0.0;
        const bool ok = attn_close(got, want, &worst);
        if (!ok) {
            std::printf("    T %u before %u: worst abs err %.3e\n", T, before, worst);
        }
        REQUIRE(ok);
        before += T;
    }
    layer.reset_cache();
    REQUIRE(mha.cache_len == 0U && mha.k_rotation.empty());
    // the other activations the constructor takes; the one it cannot run is refused
    REQUIRE(TransformerEncoderLayer(dm, H, dff, TEST_DTAG, RELU_FN).activation->mtype == RELU_T);
    REQUIRE(TransformerEncoderLayer(dm, H, dff, TEST_DTAG, SIGMOID_FN).activation->mtype == SIGMOID_T);
    REQUIRE(TransformerEncoderLayer(dm, H, dff, TEST_DTAG, TANH_FN).activation->mtype == TANH_T);
    REQUIRE_THROWS_AS(TransformerEncoderLayer(dm, H, dff, TEST_DTAG, SWIGLU_FN), std::invalid_argument);
}

TEST_CASE(test_qwen_decoder_layer_prefill_then_decode, true)
{
    // include/modules/qwen_decoder_layer.hpp:104-115: h = x + attn(rms1(x)); out = h + mlp(rms2(h)), grouped query
    // heads, rotary positions that continue across calls, the Lloyd-Max cache; a prefill, two decode steps and a
    // chunk against float64 (attention over the rows the device cache holds)
    const tcapint B = 3U, dm = 256U, H = 4U, Hkv = 2U, dff = 384U, hd = 64U;
    QwenDecoderLayer layer(dm, H, Hkv, dff, 48U);
    REQUIRE(layer.self_attn->rope && layer.self_attn->rope->max_seq_len == 48U && layer.self_attn->head_dim == (symint)hd);
    REQUIRE(layer.parameters().size() == 8U + 3U + 1U + 1U);
    MultiHeadAttention &mha = *layer.self_attn;
    mha.kv_coder = KV_LLOYDMAX;
    mha.k_bits = 3;
    mha.v_bits = 4;
    mha.gqa_blocked = true;
    mha.rotation_seed = 99U;
    const HostLinear wq = install(mha.W_q, 301U), wk = install(mha.W_k, 302U), wv = install(mha.W_v, 303U), wo = install(mha.W_o, 304U);
    (void)wk;
    (void)wv;
    HostLinear gate = install(layer.mlp->gate_proj, 305U), up = install(layer.mlp->up_proj, 307U), down = install(layer.mlp->down_proj, 309U);
    for (HostLinear *l : { &gate, &up, &down }) {
        std::fill(l->b.begin(), l->b.end(), 0.0f); // bias-free projections (swiglu.hpp:35-37)
    }
    REQUIRE(!layer.mlp->gate_proj->bias && !layer.mlp->down_proj->bias);
    std::vector<real1> w1 = gaussian(dm, 311U, 0.2f), w2 = gaussian(dm, 312U, 0.2f);
    for (tcapint j = 0; j < dm; ++j) {
        w1[j] += 1.0f;
        w2[j] += 1.0f;
    }
    set_param(layer.input_layernorm->weight, w1, { dm });
    set_param(layer.post_attention_layernorm->weight, w2, { dm });
    tcapint before = 0U;
    for (const tcapint T : { 9U, 1U, 1U, 4U }) {
        const std::vector<real1> xv = gaussian((size_t)B * T * dm, 400U + before);
        TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, dm }, false, TEST_DTAG);
        const std::vector<real1> got = layer.forward(x)->to_vector();
        REQUIRE(mha.cache_len == before + T && mha.max_seq_len == 48U);
        const size_t rows = (size_t)B * T;
        const std::vector<double> xd = to_double(xv);
        const std::vector<double> h = plus(xd, host_mha(mha, wq, wo, host_rms_norm(xd, rows, dm, w1), B, T, before));
        const std::vector<double> r2 = host_rms_norm(h, rows, dm, w2);
        const std::vector<double> gd = host_linear(gate, r2, rows), ud = host_linear(up, r2, rows);
        std::vector<double> act(gd.size());
        for (size_t i = 0; i < gd.size(); ++i) {
            act[i] = gd[i] / (1.0 + std::exp(-gd[i])) * ud[i];
        }
        const std::vector<double> want = plus(h, host_linear(down, act, rows));
        double worst = 0.0;
        const bool ok = attn_close(got, want, &worst);
        if (!ok) {
            std::printf("    T %u before %u: worst abs err %.3e\n", T, before, worst);
        }
        REQUIRE(ok);
        before += T;
    }
    // lifecycle calls reach the attention module (qwen_decoder_layer.hpp:98-102)
    layer.reset_cache();
    REQUIRE(mha.cache_len == 0U && mha.max_seq_len == 0U);
    layer.set_max_kv_seq_len(20U);
    REQUIRE(mha.max_seq_len == 20U);
}

TEST_CASE(test_projections_side_by_side, true)
{
    // fuse_projections() moves the weights of the projections that share their input (Q, K, V; gate, up) side by side
    // and runs them as one product: the same parameters, the same stream on save, results equal to those of the
    // separate products up to the rounding of a differently cut sum
    const tcapint B = 3U;
    auto close_to = [](const std::vector<real1> &a, const std::vector<real1> &b) {
        if (a.size() != b.size()) {
            return false;
        }
        for (size_t i = 0; i < a.size(); ++i) {
            if (std::fabs((double)a[i] - (double)b[i]) > std::max(1e-4, 1e-3 * std::fabs((double)b[i]))) {
                return false;
            }
        }
        return true;
    };
    {
        QwenDecoderLayer a(128U, 4U, 2U, 192U, 24U);
        a.self_attn->kv_coder = KV_LLOYDMAX;
        a.self_attn->k_bits = 3;
        a.self_attn->v_bits = 4;
        a.self_attn->rotation_seed = 8U;
        std::stringstream ss;
        a.save(ss);
        a.self_attn->save_quantizer(ss);
        const std::string before = ss.str();
        QwenDecoderLayerPtr b = std::dynamic_pointer_cast<QwenDecoderLayer>(Module::load(ss));
        REQUIRE((bool)b);
        if (!b) {
            return;
        }
        b->self_attn->load_quantizer(ss);
        std::vector<std::vector<real1>> values;
        for (const ParameterPtr &p : b->parameters()) {
            values.push_back(p->to_vector());
        }
        const std::vector<ParameterPtr> held = b->parameters();
        b->fuse_projections();
        b->fuse_projections(); // (a second call finds them in place)
        // one storage under Q, K, V and one under gate, up; the parameter objects are the ones held before
        REQUIRE(b->self_attn->W_q->weight->storage == b->self_attn->W_k->weight->storage);
        REQUIRE(b->self_attn->W_k->weight->storage == b->self_attn->W_v->weight->storage);
        REQUIRE(b->self_attn->W_q->weight->storage != b->self_attn->W_o->weight->storage);
        REQUIRE(b->mlp->gate_proj->weight->storage == b->mlp->up_proj->weight->storage);
        REQUIRE(b->self_attn->W_k->weight->offset == 128U * 128U && b->self_attn->W_v->weight->offset == 128U * (128U + 64U));
        const std::vector<ParameterPtr> now = b->parameters();
        REQUIRE(now.size() == held.size());
        for (size_t i = 0; i < now.size() && i < held.size(); ++i) {
            REQUIRE(now[i] == held[i]);
            REQUIRE(now[i]->to_vector() == values[i]);
        }
        // the stream of the moved module is the stream of the original
        std::stringstream after;
        b->save(after);
        b->self_attn->save_quantizer(after);
        REQUIRE(after.str() == before);
        tcapint seen = 0U;
        for (const tcapint T : { 6U, 1U, 1U, 3U }) {
            const std::vector<real1> xv = gaussian((size_t)B * T * 128U, 700U + seen);
            TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, 128U }, false, TEST_DTAG);
            const std::vector<real1> ya = a.forward(x)->to_vector(), yb = b->forward(x)->to_vector();
            REQUIRE(close_to(yb, ya));
            seen += T;
        }
    }
    {
        // with biases (the encoder layer's attention), and a module whose projections differ in width
        TransformerEncoderLayer a(64U, 4U, 96U, TEST_DTAG, GELU_FN);
        a.self_attn->rotation_seed = 3U;
        a.set_max_kv_seq_len(16U);
        std::stringstream ss;
        a.save(ss);
        TransformerEncoderLayerPtr b = std::dynamic_pointer_cast<TransformerEncoderLayer>(Module::load(ss));
        REQUIRE((bool)b);
        if (!b) {
            return;
        }
        b->self_attn->rotation_seed = 3U;
        b->set_max_kv_seq_len(16U);
        b->fuse_projections();
        REQUIRE(b->self_attn->W_q->bias && b->self_attn->W_q->bias->storage == b->self_attn->W_v->bias->storage);
        for (const tcapint T : { 5U, 1U }) {
            const std::vector<real1> xv = gaussian((size_t)B * T * 64U, 800U + T);
            TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, 64U }, false, TEST_DTAG);
            REQUIRE(close_to(b->forward(x)->to_vector(), a.forward(x)->to_vector()));
        }
        // modules that cannot lie side by side are refused
        LinearPtr p = std::make_shared<Linear>(8U, 4U, true, true, DType::REAL, TEST_DTAG);
        LinearPtr q = std::make_shared<Linear>(16U, 4U, true, true, DType::REAL, TEST_DTAG);
        LinearPtr r = std::make_shared<Linear>(8U, 6U, false, true, DType::REAL, TEST_DTAG);
        REQUIRE_THROWS_AS(place_side_by_side({ p, q }), std::invalid_argument);
        REQUIRE_THROWS_AS(place_side_by_side({ p, r }), std::invalid_argument);
        // ... and ones that do not (yet) are applied one by one
        LinearPtr s2 = std::make_shared<Linear>(8U, 6U, true, true, DType::REAL, TEST_DTAG);
        const std::vector<real1> xv = gaussian(5U * 8U, 9U);
        TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ 5U, 8U }, false, TEST_DTAG);
        const std::vector<TensorPtr> apart = forward_side_by_side({ p, s2 }, x);
        REQUIRE(apart.size() == 2U && apart[0]->to_vector() == p->forward(x)->to_vector());
        place_side_by_side({ p, s2 });
        const std::vector<TensorPtr> together = forward_side_by_side({ p, s2 }, x);
        REQUIRE(together.size() == 2U && together[1]->shape == std::vector<tcapint>({ 5U, 6U }));
        REQUIRE(close_to(together[0]->to_vector(), apart[0]->to_vector()));
        REQUIRE(close_to(together[1]->to_vector(), apart[1]->to_vector()));
    }
}

TEST_CASE(test_checkpoint_layers_round_trip, true)
{
    // save -> load of both layer modules (transformer_encoder_layer.cpp:126-138, qwen_decoder_layer.cpp:18-27,
    // module.cpp:231-304) and bit-identical replay of a prefill and a decode step; the fixed-size head of each record
    // against hand-assembled bytes
    const tcapint B = 2U;
    {
        TransformerEncoderLayer a(32U, 2U, 48U, TEST_DTAG, TANH_FN);
        a.self_attn->rotation_seed = 5U;
        a.set_max_kv_seq_len(16U);
        const std::vector<real1> x0 = gaussian((size_t)B * 5U * 32U, 1U), x1 = gaussian((size_t)B * 32U, 2U);
        TensorPtr t0 = std::make_shared<Tensor>(x0, std::vector<tcapint>{ B, 5U, 32U }, false, TEST_DTAG);
        TensorPtr t1 = std::make_shared<Tensor>(x1, std::vector<tcapint>{ B, 1U, 32U }, false, TEST_DTAG);
        const std::vector<real1> y0 = a.forward(t0)->to_vector(), y1 = a.forward(t1)->to_vector();
        std::stringstream ss;
        a.save(ss);
        a.self_attn->save_quantizer(ss);
        const std::string head = Bytes().u32(18U).u32(32U).u32(48U).u32(2U).u32(17U).b; // tag, d_model, d_ff, heads, attention tag
        REQUIRE(ss.str().compare(0, head.size(), head) == 0);
        TransformerEncoderLayerPtr b = std::dynamic_pointer_cast<TransformerEncoderLayer>(Module::load(ss));
        REQUIRE((bool)b);
        if (b) {
            b->self_attn->load_quantizer(ss);
            REQUIRE(ss.peek() == std::char_traits<char>::eof());
            REQUIRE(b->d_model == 32U && b->d_ff == 48U && b->num_heads == 2U && b->activation->mtype == TANH_T);
            REQUIRE(b->parameters().size() == a.parameters().size());
            REQUIRE(b->forward(t0)->to_vector() == y0);
            REQUIRE(b->forward(t1)->to_vector() == y1);
        }
    }
    {
        QwenDecoderLayer a(64U, 2U, 1U, 96U, 24U);
        a.self_attn->kv_coder = KV_LLOYDMAX;
        a.self_attn->k_bits = 2;
        a.self_attn->k_sign = true;
        a.self_attn->v_bits = 3;
        a.self_attn->rotation_seed = 6U;
        const std::vector<real1> x0 = gaussian((size_t)B * 7U * 64U, 3U), x1 = gaussian((size_t)B * 64U, 4U);
        TensorPtr t0 = std::make_shared<Tensor>(x0, std::vector<tcapint>{ B, 7U, 64U }, false, TEST_DTAG);
        TensorPtr t1 = std::make_shared<Tensor>(x1, std::vector<tcapint>{ B, 1U, 64U }, false, TEST_DTAG);
        const std::vector<real1> y0 = a.forward(t0)->to_vector(), y1 = a.forward(t1)->to_vector();
        std::stringstream ss;
        a.save(ss);
        a.self_attn->save_quantizer(ss);
        const std::string head = Bytes().u32(33U).u32(64U).u32(2U).u32(1U).u32(17U).b; // tag, d_model, heads, kv heads, attention tag
        REQUIRE(ss.str().compare(0, head.size(), head) == 0);
        QwenDecoderLayerPtr b = std::dynamic_pointer_cast<QwenDecoderLayer>(Module::load(ss));
        REQUIRE((bool)b);
        if (b) {
            b->self_attn->load_quantizer(ss);
            REQUIRE(ss.peek() == std::char_traits<char>::eof());
            REQUIRE(b->d_model == 64U && b->num_heads == 2U && b->num_kv_heads == 1U && b->self_attn->rope &&
                b->self_attn->rope->max_seq_len == 24U && b->mlp->intermediate_size == 96U);
            REQUIRE(b->input_layernorm->hidden_size == 64U && b->post_attention_layernorm->axis == -1);
            REQUIRE(b->parameters().size() == a.parameters().size());
            REQUIRE(b->forward(t0)->to_vector() == y0);
            REQUIRE(b->forward(t1)->to_vector() == y1);
        }
    }
}

TEST_CASE(test_replaced_tables_travel_in_the_quantizer_record, true)
{
    // MultiHeadAttention::set_tables forwards to weed_hip_kv_cache_set_tables; the tables are part of the quantizer
    // record, so a reloaded module codes the same tokens into the same cache rows
    const tcapint B = 2U, dm = 64U, H = 2U, Hkv = 2U, hd = 32U, T = 6U;
    auto make = [&]() {
        MultiHeadAttentionPtr m = std::make_shared<MultiHeadAttention>(dm, H, Hkv, hd, TEST_DTAG, nullptr, ZERO_R1, -1, true, 4);
        m->kv_coder = KV_LLOYDMAX;
        m->k_bits = 2;
        m->k_sign = true;
        m->v_bits = 3;
        m->rotation_seed = 77U;
        m->set_max_kv_seq_len(16U);
        return m;
    };
    // the caller's own tables: uniform grids instead of the Lloyd-Max levels (values exactly representable in binary16)
    const std::vector<real1> kb{ -1.0f, 0.0f, 1.0f }, kl{ -1.5f, -0.5f, 0.5f, 1.5f },
        kr{ -1.75f, -1.25f, -0.75f, -0.25f, 0.25f, 0.75f, 1.25f, 1.75f };
    std::vector<real1> vb, vl;
    for (int i = 0; i < 8; ++i) {
        vl.push_back(-1.75f + 0.5f * (real1)i);
        if (i) {
            vb.push_back(-2.0f + 0.5f * (real1)i);
        }
    }
    MultiHeadAttentionPtr a = make(), stock = make();
    REQUIRE_THROWS_AS(a->set_tables(0, kb, kl, kl), std::invalid_argument); // 2 bits + sign needs 8 reconstruction values
    REQUIRE_THROWS_AS(a->set_tables(2, kb, kl, kr), std::invalid_argument);
    a->set_tables(0, kb, kl, kr);
    a->set_tables(1, vb, vl, vl);
    for (const MultiHeadAttentionPtr &m : { a, stock }) {
        install(m->W_q, 1U);
        install(m->W_k, 2U);
        install(m->W_v, 3U);
        install(m->W_o, 4U);
    }
    const std::vector<real1> xv = gaussian((size_t)B * T * dm, 9U);
    TensorPtr x = std::make_shared<Tensor>(xv, std::vector<tcapint>{ B, T, dm }, false, TEST_DTAG);
    const std::vector<real1> ya = a->forward(x)->to_vector(), ys = stock->forward(x)->to_vector();
    REQUIRE(ya != ys);
    REQUIRE_THROWS_AS(a->set_tables(0, kb, kl, kr), std::logic_error); // tokens are cached
    auto rows_of = [&](MultiHeadAttention &m) {
        std::vector<real1> r((size_t)2U * B * Hkv * T * hd);
        size_t at = 0;
        for (QuantizedKVCache *qc : { &m.k_qcache, &m.v_qcache }) {
            for (tcapint p = 0; p < B * Hkv; ++p) {
                for (tcapint tok = 0; tok < T; ++tok, at += hd) {
                    qc->read_row(p * m.max_seq_len + tok, &r[at]);
                }
            }
        }
        return r;
    };
    const std::vector<real1> rows_a = rows_of(*a);
    // every dequantised coordinate is row scale times one of the caller's values: ratios of a row are ratios of table entries
    REQUIRE(rows_a != rows_of(*stock));
    std::stringstream ss;
    a->save(ss);
    a->save_quantizer(ss);
    MultiHeadAttentionPtr b = std::dynamic_pointer_cast<MultiHeadAttention>(Module::load(ss));
    REQUIRE((bool)b);
    if (!b) {
        return;
    }
    b->load_quantizer(ss);
    REQUIRE(ss.peek() == std::char_traits<char>::eof());
    REQUIRE(b->custom_tables[0].bounds == kb && b->custom_tables[0].recon == kr && b->custom_tables[1].levels == vl);
    REQUIRE(b->forward(x)->to_vector() == ya);
    REQUIRE(rows_of(*b) == rows_a);
    // the tables survive reset_cache(), as the weights do
    b->reset_cache();
    b->rotation_seed = 77U;
    b->set_max_kv_seq_len(16U);
    REQUIRE(b->forward(x)->to_vector() == ya);
    // a version-1 record (no tables) still loads: built-in tables
    std::stringstream s1;
    stock->save_quantizer(s1);
    std::string v1 = s1.str();
    REQUIRE(v1.size() > 24U && v1[3] == '2');
    v1[3] = '1';
    v1.resize(v1.size() - 24U); // six empty lists
    std::istringstream is1(v1);
    MultiHeadAttentionPtr c = make();
    c->load_quantizer(is1);
    REQUIRE(is1.peek() == std::char_traits<char>::eof());
    REQUIRE(c->custom_tables[0].bounds.empty() && c->k_rotation == stock->k_rotation);
    // the uniform coder has no tables
    MultiHeadAttention u(dm, H, Hkv, hd, TEST_DTAG, nullptr, ZERO_R1, -1, true, 4);
    REQUIRE_THROWS_AS(u.set_tables(0, kb, kl, kr), std::invalid_argument);
}

} // namespace

int main(int argc, char **argv)
{
    bool gpu = true;
    const char *filter = nullptr;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--no-gpu")) {
            gpu = false;
        } else {
            filter = argv[i];
        }
    }
    int ran = 0, failed_cases = 0;
    for (const Case &c : cases()) {
        if ((c.needs_gpu && !gpu) || (filter && !std::strstr(c.name, filter))) {
            continue;
        }
        std::printf("[ RUN  ] %s\n", c.name);
        std::fflush(stdout);
        const int before = failures;
        try {
            c.body();
        } catch (const std::exception &e) {
            std::printf("    FAILED: unexpected exception: %s\n", e.what());
            ++failures;
        }
        ++ran;
        if (failures != before) {
            ++failed_cases;
            std::printf("[ FAIL ] %s\n", c.name);
        } else {
            std::printf("[  OK  ] %s\n", c.name);
        }
        std::fflush(stdout);
    }
    if (gpu) {
        HipDevice::Instance().finish();
    }
    std::printf("%d case(s) run, %d failed\n", ran, failed_cases);
    return failed_cases ? 1 : 0;
}
