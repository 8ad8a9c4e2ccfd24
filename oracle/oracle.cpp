// CPU oracle: a restatement of the altius interpreter's tensor kernels.
// Test infrastructure only -- see oracle.h for the scope, the reference
// citations and the parity status of each function.
//
// Build with -ffp-contract=off: the reference never contracts a*b+c except
// where it writes mul_add, and those places use fmaf() here.

#include "oracle.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace {

// ---------------------------------------------------------------------------
// ThreadCtx (crates/session_interpreter/src/thread.rs:7-142): a fixed pool,
// `spawn` runs inline when the pool has one thread, `scope` ends with a join.
// ---------------------------------------------------------------------------
class Pool {
public:
    explicit Pool(size_t n) : stop_(false), pending_(0) {
        for (size_t i = 0; i < n; i++) workers_.emplace_back([this] { loop(); });
    }
    ~Pool() {
        {
            std::lock_guard<std::mutex> g(m_);
            stop_ = true;
        }
        cv_.notify_all();
        for (auto &w : workers_) w.join();
    }
    size_t size() const { return workers_.size(); }
    void execute(std::function<void()> f) {
        {
            std::lock_guard<std::mutex> g(m_);
            q_.push_back(std::move(f));
            pending_++;
        }
        cv_.notify_one();
    }
    void join() {
        std::unique_lock<std::mutex> g(m_);
        done_.wait(g, [this] { return pending_ == 0; });
    }

private:
    void loop() {
        for (;;) {
            std::function<void()> f;
            {
                std::unique_lock<std::mutex> g(m_);
                cv_.wait(g, [this] { return stop_ || !q_.empty(); });
                if (stop_ && q_.empty()) return;
                f = std::move(q_.back());
                q_.pop_back();
            }
            f();
            {
                std::lock_guard<std::mutex> g(m_);
                if (--pending_ == 0) done_.notify_all();
            }
        }
    }
    std::vector<std::thread> workers_;
    std::vector<std::function<void()>> q_;
    std::mutex m_;
    std::condition_variable cv_, done_;
    bool stop_;
    size_t pending_;
};

std::mutex g_pool_mutex;
Pool *g_pool = nullptr;

Pool *pool_for(size_t n) {
    std::lock_guard<std::mutex> g(g_pool_mutex);
    if (!g_pool || g_pool->size() != n) {
        delete g_pool;
        g_pool = new Pool(n);
    }
    return g_pool;
}

struct Scope {
    size_t n;
    Pool *pool;
    explicit Scope(int threads) : n(threads < 1 ? 1 : (size_t)threads), pool(nullptr) {
        if (n > 1) pool = pool_for(n);
    }
    template <class F> void spawn(F &&f) {
        if (n == 1)
            f();
        else
            pool->execute(std::function<void()>(std::forward<F>(f)));
    }
    void join() {
        if (n != 1) pool->join();
    }
};

// ---------------------------------------------------------------------------
// Scalar helpers with Rust semantics.
// ---------------------------------------------------------------------------
inline uint32_t bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float from_bits(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
// f32::max / Simd::simd_max: the non-NaN operand wins.
inline float rmax(float v, float m) { return (m != m || v > m) ? v : m; }
// f32::clamp / Simd::simd_clamp: NaN passes through, comparisons only.
inline float rclamp(float x, float lo, float hi) {
    if (x < lo) x = lo;
    if (x > hi) x = hi;
    return x;
}

constexpr size_t SIMD_LEN = 8;

// Simd::reduce_sum: ordered, lanes 0..7, starting from -0.0.
inline float reduce_sum8(const float *acc) {
    float s = -0.0f;
    for (size_t k = 0; k < SIMD_LEN; k++) s += acc[k];
    return s;
}

// session.rs:1028-1040
float fast_sum(const float *x, size_t len) {
    float acc[SIMD_LEN] = {0, 0, 0, 0, 0, 0, 0, 0};
    while (len >= SIMD_LEN) {
        for (size_t k = 0; k < SIMD_LEN; k++) acc[k] += x[k];
        x += SIMD_LEN;
        len -= SIMD_LEN;
    }
    float tail = -0.0f;  // Iterator::sum::<f32>() folds from -0.0
    for (size_t i = 0; i < len; i++) tail += x[i];
    return reduce_sum8(acc) + tail;
}

// session.rs:1042-1055
float fast_sum_squares(const float *x, size_t len) {
    float acc[SIMD_LEN] = {0, 0, 0, 0, 0, 0, 0, 0};
    while (len >= SIMD_LEN) {
        for (size_t k = 0; k < SIMD_LEN; k++) acc[k] += x[k] * x[k];
        x += SIMD_LEN;
        len -= SIMD_LEN;
    }
    float tail = -0.0f;
    for (size_t i = 0; i < len; i++) tail += x[i] * x[i];
    return reduce_sum8(acc) + tail;
}

// ---------------------------------------------------------------------------
// fast_math.rs
// ---------------------------------------------------------------------------
constexpr float ROUNDING_BIAS = 12582912.0f;
constexpr float LOG2RECIPROCAL = 1.44269504088896341f;
constexpr float LOG2HIGH = -6.93145752e-1f;
constexpr float LOG2LOW = -1.42860677e-6f;
constexpr float POLY_0 = 0.0013780593872f;
constexpr float POLY_1 = 0.0083731245250f;
constexpr float POLY_2 = 0.0416695363820f;
constexpr float POLY_3 = 0.1666647195816f;
constexpr float POLY_4 = 0.4999998509884f;
constexpr float POLY_56 = 1.0000000000000f;
constexpr int32_t MINIMUM_EXPONENT = -1056964608;
constexpr int32_t MAXIMUM_EXPONENT = 0x3F800000;

// One element of fast_sum_exp (fast_math.rs:130-150 / 161-180).
inline float sum_exp_elem(float x, float max) {
    const float LOWER_RANGE_2 = -88.37626f;
    float v = rmax(x - max, LOWER_RANGE_2);
    float biased = fmaf(v, LOG2RECIPROCAL, ROUNDING_BIAS);
    float m = biased - ROUNDING_BIAS;
    v = fmaf(m, LOG2HIGH, v);
    v = fmaf(m, LOG2LOW, v);
    uint32_t normal = (bits(biased) << 23) + (uint32_t)MAXIMUM_EXPONENT;
    float p = POLY_0;
    p = fmaf(p, v, POLY_1);
    p = fmaf(p, v, POLY_2);
    p = fmaf(p, v, POLY_3);
    p = fmaf(p, v, POLY_4);
    p = fmaf(p, v, POLY_56);
    p = fmaf(p, v, POLY_56);
    return p * from_bits(normal);
}

// fast_math.rs:102-187
float fast_sum_exp(float *out, const float *in, size_t len) {
    float max = NAN;
    for (size_t i = 0; i < len; i++) max = rmax(in[i], max);

    float acc[SIMD_LEN] = {0, 0, 0, 0, 0, 0, 0, 0};
    while (len >= SIMD_LEN) {
        float p[SIMD_LEN];
        for (size_t k = 0; k < SIMD_LEN; k++) p[k] = sum_exp_elem(in[k], max);
        for (size_t k = 0; k < SIMD_LEN; k++) acc[k] += p[k];
        for (size_t k = 0; k < SIMD_LEN; k++) out[k] = p[k];
        in += SIMD_LEN;
        out += SIMD_LEN;
        len -= SIMD_LEN;
    }
    float sum = reduce_sum8(acc);
    for (size_t i = 0; i < len; i++) {
        float p = sum_exp_elem(in[i], max);
        sum += p;
        out[i] = p;
    }
    return sum;
}

// One element of fast_sigmoid (fast_math.rs:214-244 / 251-277).
inline float sigmoid_elem(float x) {
    const float LOWER_RANGE = -103.9720840454f;
    const float UPPER_RANGE = 88.7762626647950f;
    float v = rclamp(-x, LOWER_RANGE, UPPER_RANGE);
    float biased = fmaf(v, LOG2RECIPROCAL, ROUNDING_BIAS);
    float m = biased - ROUNDING_BIAS;
    v = fmaf(m, LOG2HIGH, v);
    v = fmaf(m, LOG2LOW, v);
    int32_t overflow = (int32_t)(bits(biased) << 23);
    int32_t normal = overflow < MAXIMUM_EXPONENT ? overflow : MAXIMUM_EXPONENT;
    normal = normal > MINIMUM_EXPONENT ? normal : MINIMUM_EXPONENT;
    uint32_t of = (uint32_t)overflow - (uint32_t)normal + (uint32_t)MAXIMUM_EXPONENT;
    uint32_t nf = (uint32_t)normal + (uint32_t)MAXIMUM_EXPONENT;
    float p = POLY_0;
    p = fmaf(p, v, POLY_1);
    p = fmaf(p, v, POLY_2);
    p = fmaf(p, v, POLY_3);
    p = fmaf(p, v, POLY_4);
    p = fmaf(p, v, POLY_56);
    v = v * from_bits(of);
    p = fmaf(p, v, from_bits(of));
    p = p * from_bits(nf);
    return 1.0f / (1.0f + p);
}

// fast_math.rs:189-279 (the 8-lane body and the scalar tail compute the same
// per-element expression, so one loop restates both).
void fast_sigmoid(float *out, const float *in, size_t len) {
    for (size_t i = 0; i < len; i++) out[i] = sigmoid_elem(in[i]);
}

// One element of fast_gelu (fast_math.rs:304-323 / 332-353).
inline float gelu_elem(float i) {
    const float B = 0.7978845608028654f;
    const float C = 0.035677408136300125f;
    const float ALPHA_13 = -2.76076847742355e-16f;
    const float ALPHA_11 = 2.00018790482477e-13f;
    const float ALPHA_9 = -8.60467152213735e-11f;
    const float ALPHA_7 = 5.12229709037114e-08f;
    const float ALPHA_5 = 1.48572235717979e-05f;
    const float ALPHA_3 = 6.37261928875436e-04f;
    const float ALPHA_1 = 4.89352455891786e-03f;
    const float BETA_6 = 1.19825839466702e-06f;
    const float BETA_4 = 1.18534705686654e-04f;
    const float BETA_2 = 2.26843463243900e-03f;
    const float BETA_0 = 4.89352518554385e-03f;

    float v = i * (C * i * i + B);  // plain mul/add, no fma (fast_math.rs:305,333)
    v = rclamp(v, -9.0f, 9.0f);
    float v2 = v * v;
    float p = fmaf(v2, ALPHA_13, ALPHA_11);
    p = fmaf(p, v2, ALPHA_9);
    p = fmaf(p, v2, ALPHA_7);
    p = fmaf(p, v2, ALPHA_5);
    p = fmaf(p, v2, ALPHA_3);
    p = fmaf(p, v2, ALPHA_1);
    p = p * v;
    float q = fmaf(v2, BETA_6, BETA_4);
    q = fmaf(q, v2, BETA_2);
    q = fmaf(q, v2, BETA_0);
    float o = p / q;
    return (o + 1.0f) * (i * 0.5f);
}

// One element of tanh (session.rs:860-877 / 883-902): the same 13/6-degree
// rational function fast_gelu uses, on the clamped input itself.
inline float tanh_elem(float x) {
    const float ALPHA_13 = -2.76076847742355e-16f;
    const float ALPHA_11 = 2.00018790482477e-13f;
    const float ALPHA_9 = -8.60467152213735e-11f;
    const float ALPHA_7 = 5.12229709037114e-08f;
    const float ALPHA_5 = 1.48572235717979e-05f;
    const float ALPHA_3 = 6.37261928875436e-04f;
    const float ALPHA_1 = 4.89352455891786e-03f;
    const float BETA_6 = 1.19825839466702e-06f;
    const float BETA_4 = 1.18534705686654e-04f;
    const float BETA_2 = 2.26843463243900e-03f;
    const float BETA_0 = 4.89352518554385e-03f;
    float v = rclamp(x, -9.0f, 9.0f);
    float v2 = v * v;
    float p = fmaf(v2, ALPHA_13, ALPHA_11);
    p = fmaf(p, v2, ALPHA_9);
    p = fmaf(p, v2, ALPHA_7);
    p = fmaf(p, v2, ALPHA_5);
    p = fmaf(p, v2, ALPHA_3);
    p = fmaf(p, v2, ALPHA_1);
    p = p * v;
    float q = fmaf(v2, BETA_6, BETA_4);
    q = fmaf(q, v2, BETA_2);
    q = fmaf(q, v2, BETA_0);
    return p / q;
}

void fast_gelu(float *out, const float *in, size_t len) {
    for (size_t i = 0; i < len; i++) out[i] = gelu_elem(in[i]);
}

// fastapprox 0.3.1, module `faster` (not vendored in the reference; restated
// from the crate's published algorithm; only the fitted constant K stays unconfirmed, see oracle.h):
//   pow2(p) = from_bits(((1 << 23) as f32 * (max(p, -126) + 126.94269504)) as u32)
//   erfc(x) = 2 / (1 + pow2(3.3509633149424609 * x));  erf(x) = 1 - erfc(x)
// Rust's `as u32` saturates and maps NaN to 0.
inline uint32_t f32_as_u32_saturating(float f) {
    if (!(f > 0.0f)) return 0u;  // negative, zero, NaN
    if (f >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)f;
}
inline float faster_pow2(float p) {
    float clipp = p < -126.0f ? -126.0f : p;
    return from_bits(f32_as_u32_saturating((float)(1 << 23) * (clipp + 126.94269504f)));
}
inline float faster_erf(float x) {
    const float K = 3.3509633149424609f;
    float erfc = 2.0f / (1.0f + faster_pow2(K * x));
    return 1.0f - erfc;
}

// ---------------------------------------------------------------------------
// Shapes.
// ---------------------------------------------------------------------------
using Dims = std::vector<int64_t>;

bool is_scalar(const Dims &d) { return d.empty() || (d.size() == 1 && (d[0] == 0 || d[0] == 1)); }

int64_t total_elems(const Dims &d) {
    int64_t n = 1;
    for (auto v : d) n *= v;
    return n;
}

Dims compute_strides(const Dims &d) {
    Dims s(d.size());
    for (size_t i = 0; i < d.size(); i++) {
        int64_t p = 1;
        for (size_t j = i + 1; j < d.size(); j++) p *= d[j];
        s[i] = p;
    }
    return s;
}

// fixed_dim.rs:112-136
bool broadcast(const std::vector<Dims> &shapes, Dims *out) {
    if (shapes.empty()) return false;
    size_t max_len = 0;
    for (auto &s : shapes) max_len = s.size() > max_len ? s.size() : max_len;
    Dims shape;
    for (size_t i = 0; i < max_len; i++) {
        int64_t size = 1;
        for (auto &s : shapes) {
            size_t len = s.size();
            int64_t dim = i < len ? s[len - i - 1] : 1;
            if (dim == 1) continue;
            if (size != 1 && dim != size) return false;
            size = dim;
        }
        shape.push_back(size);
    }
    out->assign(shape.rbegin(), shape.rend());
    return true;
}

// tensor.rs:369-406
bool strides_for_broadcasting(const Dims &from, const Dims &to, Dims *out) {
    Dims stride = compute_strides(from);
    Dims ns = to;
    if (to.size() < from.size()) return false;
    size_t nf = from.size(), nt = to.size();
    for (size_t i = 0; i < nf; i++) {
        int64_t er = from[nf - 1 - i];
        int64_t es = stride[nf - 1 - i];
        int64_t &dr = ns[nt - 1 - i];
        if (dr == er)
            dr = es;
        else if (er == 1)
            dr = 0;
        else
            return false;
    }
    for (size_t i = nf; i < nt; i++) ns[nt - 1 - i] = 0;
    *out = ns;
    return true;
}

// ---------------------------------------------------------------------------
// Binary ops (session.rs:384-526).
// ---------------------------------------------------------------------------
struct OpAdd { static inline float f(float a, float b) { return a + b; } };
struct OpSub { static inline float f(float a, float b) { return a - b; } };
struct OpMul { static inline float f(float a, float b) { return a * b; } };
struct OpDiv { static inline float f(float a, float b) { return a / b; } };
struct OpPow { static inline float f(float a, float b) { return powf(a, b); } };

// session.rs:446-507: recursion over axes with the innermost loop specialised
// on the (a_stride, b_stride) pair.
template <class OP>
void general_compute(const int64_t *a_stride, const int64_t *b_stride, const int64_t *o_stride,
                     const int64_t *o_shape, size_t rank, const float *a, const float *b, float *o) {
    if (rank == 1) {
        int64_t len = o_shape[0];
        int64_t as = a_stride[0], bs = b_stride[0];
        if (as == 1 && bs == 1) {
            for (int64_t i = 0; i < len; i++) o[i] = OP::f(a[i], b[i]);
            return;
        }
        if (as == 0 && bs == 0) {
            float av = a[0], bv = b[0];
            for (int64_t i = 0; i < len; i++) o[i] = OP::f(av, bv);
            return;
        }
        if (as == 1 && bs == 0) {
            float bv = b[0];
            for (int64_t i = 0; i < len; i++) o[i] = OP::f(a[i], bv);
            return;
        }
        if (as == 0 && bs == 1) {
            float av = a[0];
            for (int64_t i = 0; i < len; i++) o[i] = OP::f(av, b[i]);
            return;
        }
        for (int64_t i = 0; i < len; i++) {
            o[i] = OP::f(a[0], b[0]);
            a += as;
            b += bs;
        }
        return;
    }
    for (int64_t i = 0; i < o_shape[0]; i++)
        general_compute<OP>(a_stride + 1, b_stride + 1, o_stride + 1, o_shape + 1, rank - 1,
                            a + i * a_stride[0], b + i * b_stride[0], o + i * o_stride[0]);
}

template <class OP>
int binary_general(const float *a, const Dims &ad, const float *b, const Dims &bd, float *out,
                   const Dims &od) {
    Dims as, bs;
    if (!strides_for_broadcasting(ad, od, &as) || !strides_for_broadcasting(bd, od, &bs))
        return ORC_ERR_BROADCAST;
    Dims os = compute_strides(od);
    if (total_elems(od) == 0) return ORC_OK;
    general_compute<OP>(as.data(), bs.data(), os.data(), od.data(), od.size(), a, b, out);
    return ORC_OK;
}

template <class OP>
int binary_elemwise(const float *a, const Dims &ad, const float *b, const Dims &bd, float *out,
                    int threads, int strict) {
    if (ad == bd) {  // session.rs:394-418
        size_t n = (size_t)total_elems(ad);
        const size_t chunk = 100000;
        Scope scope(threads);
        for (size_t s = 0; s < n; s += chunk) {
            size_t e = s + chunk < n ? s + chunk : n;
            scope.spawn([=] {
                for (size_t i = s; i < e; i++) out[i] = OP::f(a[i], b[i]);
            });
        }
        scope.join();
        return ORC_OK;
    }
    if (is_scalar(bd)) {  // session.rs:420-429
        float bv = b[0];
        size_t n = (size_t)total_elems(ad);
        for (size_t i = 0; i < n; i++) out[i] = OP::f(a[i], bv);
        return ORC_OK;
    }
    if (is_scalar(ad)) {  // session.rs:431-440
        float av = a[0];
        size_t n = (size_t)total_elems(bd);
        for (size_t i = 0; i < n; i++) out[i] = OP::f(av, b[i]);
        return ORC_OK;
    }
    Dims od;
    if (!broadcast({ad, bd}, &od)) return ORC_ERR_BROADCAST;
    if (od.size() <= 1 && strict) return ORC_ERR_UNSUPPORTED;  // session.rs:521 assert
    return binary_general<OP>(a, ad, b, bd, out, od);
}

// session.rs:566-606
int pow_op(const float *a, const Dims &ad, const float *b, const Dims &bd, float *out, int strict,
           int *no_ref) {
    if (ad == bd) {
        size_t n = (size_t)total_elems(ad);
        for (size_t i = 0; i < n; i++) out[i] = powf(a[i], b[i]);
        return ORC_OK;
    }
    if (is_scalar(bd)) {
        float bv = b[0];
        size_t n = (size_t)total_elems(ad);
        if (bv == 2.0f) {
            for (size_t i = 0; i < n; i++) out[i] = a[i] * a[i];
        } else {
            for (size_t i = 0; i < n; i++) out[i] = powf(a[i], bv);
        }
        return ORC_OK;
    }
    // todo!() in the reference: multidirectional broadcast is not implemented.
    if (strict) return ORC_ERR_UNSUPPORTED;
    if (no_ref) *no_ref = 1;
    Dims od;
    if (!broadcast({ad, bd}, &od)) return ORC_ERR_BROADCAST;
    return binary_general<OpPow>(a, ad, b, bd, out, od);
}

// ---------------------------------------------------------------------------
// Reductions.
// ---------------------------------------------------------------------------
std::vector<size_t> normalise_axes(int rank, int n_axes, const int64_t *axes) {
    std::vector<size_t> r;
    for (int i = 0; i < n_axes; i++) r.push_back((size_t)(axes[i] < 0 ? rank + axes[i] : axes[i]));
    return r;
}

bool contains(const std::vector<size_t> &v, size_t x) {
    for (auto e : v)
        if (e == x) return true;
    return false;
}

// shape.rs:354-411
int reduce_shape(int kind, const Dims &in, int n_axes, const int64_t *axes, int keep, Dims *out) {
    std::vector<size_t> ax;
    if (kind == ORC_REDUCE_MAX && n_axes == 0) {
        for (size_t i = 0; i < in.size(); i++) ax.push_back(i);
    } else {
        ax = normalise_axes((int)in.size(), n_axes, axes);
    }
    Dims d;
    for (size_t i = 0; i < in.size(); i++) {
        if (contains(ax, i)) {
            if (keep) d.push_back(1);
        } else {
            d.push_back(in[i]);
        }
    }
    if (d.empty()) d.push_back(1);
    *out = d;
    return ORC_OK;
}

// Splits dims into (outer, reduce, inner) when the reduced axes are one
// contiguous run of axes.
bool split_contiguous(const Dims &in, const std::vector<size_t> &ax, int64_t *outer, int64_t *red,
                      int64_t *inner) {
    if (ax.empty()) return false;
    size_t lo = in.size(), hi = 0;
    for (auto a : ax) {
        if (a >= in.size()) return false;
        lo = a < lo ? a : lo;
        hi = a > hi ? a : hi;
    }
    for (size_t i = lo; i <= hi; i++)
        if (!contains(ax, i)) return false;
    *outer = *red = *inner = 1;
    for (size_t i = 0; i < lo; i++) *outer *= in[i];
    for (size_t i = lo; i <= hi; i++) *red *= in[i];
    for (size_t i = hi + 1; i < in.size(); i++) *inner *= in[i];
    return true;
}

}  // namespace

// ===========================================================================
// C interface.
// ===========================================================================
extern "C" {

int orc_is_scalar(int rank, const int64_t *dims) { return is_scalar(Dims(dims, dims + rank)); }

int orc_broadcast(int n_shapes, const int *ranks, const int64_t *const *dims, int *out_rank,
                  int64_t *out_dims) {
    std::vector<Dims> shapes;
    for (int i = 0; i < n_shapes; i++) shapes.emplace_back(dims[i], dims[i] + ranks[i]);
    Dims out;
    if (!broadcast(shapes, &out)) return ORC_ERR_BROADCAST;
    *out_rank = (int)out.size();
    for (size_t i = 0; i < out.size(); i++) out_dims[i] = out[i];
    return ORC_OK;
}

int orc_strides_for_broadcasting(int from_rank, const int64_t *from_dims, int to_rank,
                                 const int64_t *to_dims, int64_t *out_strides) {
    Dims out;
    if (!strides_for_broadcasting(Dims(from_dims, from_dims + from_rank),
                                  Dims(to_dims, to_dims + to_rank), &out))
        return ORC_ERR_BROADCAST;
    for (size_t i = 0; i < out.size(); i++) out_strides[i] = out[i];
    return ORC_OK;
}

void orc_compute_strides(int rank, const int64_t *dims, int64_t *out_strides) {
    Dims s = compute_strides(Dims(dims, dims + rank));
    for (size_t i = 0; i < s.size(); i++) out_strides[i] = s[i];
}

int orc_reduce_shape(int kind, int rank, const int64_t *dims, int n_axes, const int64_t *axes,
                     int keep_dims, int *out_rank, int64_t *out_dims) {
    Dims out;
    int rc = reduce_shape(kind, Dims(dims, dims + rank), n_axes, axes, keep_dims, &out);
    if (rc != ORC_OK) return rc;
    *out_rank = (int)out.size();
    for (size_t i = 0; i < out.size(); i++) out_dims[i] = out[i];
    return ORC_OK;
}

int orc_binary(int op, const float *a, int a_rank, const int64_t *a_dims, const float *b, int b_rank,
               const int64_t *b_dims, float *out, int threads, int strict,
               int *no_reference_kernel) {
    Dims ad(a_dims, a_dims + a_rank), bd(b_dims, b_dims + b_rank);
    if (no_reference_kernel) *no_reference_kernel = 0;
    switch (op) {
    case ORC_ADD: return binary_elemwise<OpAdd>(a, ad, b, bd, out, threads, strict);
    case ORC_SUB: return binary_elemwise<OpSub>(a, ad, b, bd, out, threads, strict);
    case ORC_MUL: return binary_elemwise<OpMul>(a, ad, b, bd, out, threads, strict);
    case ORC_DIV: return binary_elemwise<OpDiv>(a, ad, b, bd, out, threads, strict);
    case ORC_POW: return pow_op(a, ad, b, bd, out, strict, no_reference_kernel);
    }
    return ORC_ERR_ARG;
}

int orc_unary(int op, const float *in, float *out, size_t n, float alpha, float beta, int threads) {
    switch (op) {
    case ORC_SQRT:  // session.rs:608-619
        for (size_t i = 0; i < n; i++) out[i] = sqrtf(in[i]);
        return ORC_OK;
    case ORC_RELU:  // session.rs:796-803: i.max(0.0); NaN -> 0.0
        for (size_t i = 0; i < n; i++) out[i] = in[i] > 0.0f ? in[i] : 0.0f;
        return ORC_OK;
    case ORC_HARDSIGMOID:  // session.rs:805-812
        for (size_t i = 0; i < n; i++) out[i] = rclamp(fmaf(alpha, in[i], beta), 0.0f, 1.0f);
        return ORC_OK;
    case ORC_TANH:  // session.rs:933-938
        for (size_t i = 0; i < n; i++) out[i] = tanh_elem(in[i]);
        return ORC_OK;
    case ORC_ERF:  // session.rs:924-931
        for (size_t i = 0; i < n; i++) out[i] = faster_erf(in[i]);
        return ORC_OK;
    case ORC_GELU: {  // session.rs:823-838: chunks(len / n_threads)
        Scope scope(threads);
        if (n == 0) return ORC_OK;
        size_t chunk = n / scope.n;
        if (chunk == 0) return ORC_ERR_UNSUPPORTED;  // chunks(0) panics in the reference
        for (size_t s = 0; s < n; s += chunk) {
            size_t len = s + chunk < n ? chunk : n - s;
            scope.spawn([=] { fast_gelu(out + s, in + s, len); });
        }
        scope.join();
        return ORC_OK;
    }
    case ORC_SIGMOID: {  // session.rs:905-922
        Scope scope(threads);
        const size_t threshold = 512;
        size_t chunk = n / scope.n;
        if (chunk > threshold) {
            for (size_t s = 0; s < n; s += chunk) {
                size_t len = s + chunk < n ? chunk : n - s;
                scope.spawn([=] { fast_sigmoid(out + s, in + s, len); });
            }
            scope.join();
        } else {
            fast_sigmoid(out, in, n);
        }
        return ORC_OK;
    }
    }
    return ORC_ERR_ARG;
}

int orc_softmax(const float *in, float *out, size_t rows, size_t len, int threads) {
    // session.rs:1005: batch = max(total / n_threads / axis_len, 1)
    if (rows == 0 || len == 0) return ORC_OK;
    Scope scope(threads);
    size_t batch = rows * len / scope.n / len;
    if (batch < 1) batch = 1;
    for (size_t r0 = 0; r0 < rows; r0 += batch) {
        size_t r1 = r0 + batch < rows ? r0 + batch : rows;
        scope.spawn([=] {
            for (size_t r = r0; r < r1; r++) {
                float *o = out + r * len;
                float sum = fast_sum_exp(o, in + r * len, len);
                float recip_sum = 1.0f / sum;
                for (size_t i = 0; i < len; i++) o[i] *= recip_sum;
            }
        });
    }
    scope.join();
    return ORC_OK;
}

int orc_layer_norm(const float *in, const float *scale, const float *bias, float *out, size_t rows,
                   size_t len, float eps, int threads) {
    if (rows == 0 || len == 0) return ORC_OK;
    Scope scope(threads);
    size_t batch = rows * len / scope.n / len;  // session.rs:1458
    if (batch < 1) batch = 1;
    for (size_t r0 = 0; r0 < rows; r0 += batch) {
        size_t r1 = r0 + batch < rows ? r0 + batch : rows;
        scope.spawn([=] {
            for (size_t r = r0; r < r1; r++) {
                const float *x = in + r * len;
                float *o = out + r * len;
                float inv_axis_len = 1.0f / (float)len;  // (axis_len as f32).recip()
                float mean = fast_sum(x, len) * inv_axis_len;
                for (size_t i = 0; i < len; i++) o[i] = x[i] - mean;
                float inv_std =
                    1.0f / sqrtf(fmaf(fast_sum_squares(o, len), inv_axis_len, eps));
                for (size_t i = 0; i < len; i++) o[i] = fmaf(o[i] * inv_std, scale[i], bias[i]);
            }
        });
    }
    scope.join();
    return ORC_OK;
}

int orc_reduce(int kind, const float *in, int rank, const int64_t *dims, int n_axes,
               const int64_t *axes, int keep_dims, float *out, int strict,
               int *no_reference_kernel, int *saw_nan) {
    Dims d(dims, dims + rank);
    if (no_reference_kernel) *no_reference_kernel = 0;
    if (saw_nan) *saw_nan = 0;

    if (kind == ORC_REDUCE_MEAN) {
        std::vector<size_t> ax = normalise_axes(rank, n_axes, axes);
        bool is_ref = ax.size() == 1 && rank == 3 && ax[0] == 2 && keep_dims;  // session.rs:1321-1326
        if (!is_ref) {
            if (strict) return ORC_ERR_UNSUPPORTED;
            if (no_reference_kernel) *no_reference_kernel = 1;
        }
        int64_t outer, red, inner;
        if (!split_contiguous(d, ax, &outer, &red, &inner)) return ORC_ERR_UNSUPPORTED;
        if (outer * red * inner == 0) return ORC_OK;
        float r_axis_len = 1.0f / (float)red;  // session.rs:1331
        if (inner == 1) {
            for (int64_t o = 0; o < outer; o++)
                out[o] = fast_sum(in + o * red, (size_t)red) * r_axis_len;  // session.rs:1337-1338
        } else {
            // No reference kernel: sequential sum along the reduced axis.
            for (int64_t o = 0; o < outer; o++)
                for (int64_t i = 0; i < inner; i++) {
                    float s = 0.0f;
                    for (int64_t r = 0; r < red; r++) s += in[(o * red + r) * inner + i];
                    out[o * inner + i] = s * r_axis_len;
                }
        }
        return ORC_OK;
    }

    if (kind == ORC_REDUCE_MAX) {
        bool is_ref = n_axes == 0 && !keep_dims;  // session.rs:1295-1296
        std::vector<size_t> ax;
        if (n_axes == 0) {
            for (int i = 0; i < rank; i++) ax.push_back((size_t)i);
        } else {
            ax = normalise_axes(rank, n_axes, axes);
        }
        if (!is_ref) {
            if (strict) return ORC_ERR_UNSUPPORTED;
            if (no_reference_kernel) *no_reference_kernel = 1;
        }
        int64_t outer = 1, red = 1, inner = 1;
        if (rank == 0) {
            red = 1;
        } else if (!split_contiguous(d, ax, &outer, &red, &inner)) {
            return ORC_ERR_UNSUPPORTED;
        }
        if (outer * red * inner == 0) return ORC_OK;
        // session.rs:1301-1304: max_by(partial_cmp): the last of equal maxima
        // wins; a NaN makes the reference panic (reported through *saw_nan,
        // and skipped here).
        for (int64_t o = 0; o < outer; o++)
            for (int64_t i = 0; i < inner; i++) {
                bool have = false;
                float m = NAN;
                for (int64_t r = 0; r < red; r++) {
                    float v = in[(o * red + r) * inner + i];
                    if (v != v) {
                        if (saw_nan) *saw_nan = 1;
                        continue;
                    }
                    if (!have || v >= m) {
                        m = v;
                        have = true;
                    }
                }
                out[o * inner + i] = m;
            }
        return ORC_OK;
    }
    return ORC_ERR_ARG;
}

// ---- data movement (session.rs:940-988, 1134-1278, 1350-1431, 1488-1598) ----------------------

static size_t total_of(int rank, const int64_t *dims) {
    size_t n = 1;
    for (int i = 0; i < rank; i++) n *= (size_t)dims[i];
    return n;
}

// compute_transpose: blocks = the run of trailing axes with perm[i] == i; every other axis is
// walked by an odometer whose digit i advances the source by the input stride of perm[i].
int orc_transpose(const void *in, void *out, int elem_size, int rank, const int64_t *in_dims, const int64_t *perm) {
    if (rank < 0 || rank > 16 || elem_size <= 0) return ORC_ERR_ARG;
    std::vector<int64_t> in_str((size_t)rank), out_dims((size_t)rank), new_str((size_t)rank);
    int64_t acc = 1;
    for (int i = rank - 1; i >= 0; i--) {
        in_str[(size_t)i] = acc;
        acc *= in_dims[i];
    }
    for (int i = 0; i < rank; i++) {
        if (perm[i] < 0 || perm[i] >= rank) return ORC_ERR_ARG;
        out_dims[(size_t)i] = in_dims[perm[i]];
        new_str[(size_t)i] = in_str[(size_t)perm[i]];
    }
    size_t num_blocks = 1, block = 1;
    int reduced = 0;
    bool suffix = true;
    for (int i = rank - 1; i >= 0; i--) {
        const int axis = (int)perm[i];
        if (suffix && axis == i) {
            block *= (size_t)in_dims[axis];
        } else {
            suffix = false;
            num_blocks *= (size_t)in_dims[axis];
            reduced++;
        }
    }
    if (num_blocks * block == 0) return ORC_OK;
    const char *src = static_cast<const char *>(in);
    char *dst = static_cast<char *>(out);
    std::vector<size_t> index((size_t)reduced, 0);
    size_t src_idx = 0;
    for (size_t b = 0; b < num_blocks; b++) {
        std::memcpy(dst + b * block * (size_t)elem_size, src + src_idx * (size_t)elem_size, block * (size_t)elem_size);
        // next_index (session.rs:1188-1216)
        for (int pos = reduced - 1; pos >= 0; pos--) {
            src_idx += (size_t)new_str[(size_t)pos];
            index[(size_t)pos]++;
            if (index[(size_t)pos] < (size_t)out_dims[(size_t)pos]) break;
            src_idx -= (size_t)new_str[(size_t)pos] * index[(size_t)pos];
            index[(size_t)pos] = 0;
        }
    }
    return ORC_OK;
}

int orc_gather(const void *data, int elem_size, int rank, const int64_t *dims, int axis, const int64_t *indices,
               int idx_rank, const int64_t *idx_dims, void *out, int strict, int *no_reference_kernel) {
    if (axis < 0) axis += rank;
    if (axis < 0 || axis >= rank) return ORC_ERR_ARG;
    const bool scalar = orc_is_scalar(idx_rank, idx_dims) != 0;
    bool leading_ones = true;
    for (int i = 0; i < axis; i++) leading_ones = leading_ones && dims[i] == 1;
    const bool ref = (scalar && leading_ones) || (!scalar && idx_rank == 2 && idx_dims[0] == 1 && axis == 0 && rank == 2);
    if (no_reference_kernel) *no_reference_kernel = ref ? 0 : 1;
    if (!ref && strict) return ORC_ERR_UNSUPPORTED;
    size_t outer = 1, inner = 1;
    for (int i = 0; i < axis; i++) outer *= (size_t)dims[i];
    for (int i = axis + 1; i < rank; i++) inner *= (size_t)dims[i];
    const size_t axis_len = (size_t)dims[axis], n_idx = total_of(idx_rank, idx_dims);
    const char *src = static_cast<const char *>(data);
    char *dst = static_cast<char *>(out);
    const size_t row = inner * (size_t)elem_size;
    for (size_t o = 0; o < outer; o++)
        for (size_t j = 0; j < n_idx; j++) {
            int64_t k = indices[j];
            if (k < 0) k += (int64_t)axis_len;
            if (k < 0 || k >= (int64_t)axis_len) return ORC_ERR_ARG;
            std::memcpy(dst + (o * n_idx + j) * row, src + (o * axis_len + (size_t)k) * row, row);
        }
    return ORC_OK;
}

int orc_split(const void *in, int elem_size, int rank, const int64_t *dims, int axis, int n_parts,
              const int64_t *parts, void *const *outs, int strict, int *no_reference_kernel) {
    if (axis < 0) axis += rank;
    if (axis < 0 || axis >= rank) return ORC_ERR_ARG;
    const bool ref = axis == rank - 1;  // assert_eq!(axis, inputs[0].dims().len() - 1)
    if (no_reference_kernel) *no_reference_kernel = ref ? 0 : 1;
    if (!ref && strict) return ORC_ERR_UNSUPPORTED;
    size_t outer = 1, inner = 1;
    for (int i = 0; i < axis; i++) outer *= (size_t)dims[i];
    for (int i = axis + 1; i < rank; i++) inner *= (size_t)dims[i];
    const size_t axis_len = (size_t)dims[axis];
    const char *src = static_cast<const char *>(in);
    // session.rs:1500-1511: walk the rows of the split axis, dealing each part to its output.
    std::vector<size_t> offset((size_t)n_parts, 0);
    for (size_t o = 0; o < outer; o++) {
        size_t s = 0;
        for (int p = 0; p < n_parts; p++) {
            const size_t bytes = (size_t)parts[p] * inner * (size_t)elem_size;
            std::memcpy(static_cast<char *>(outs[p]) + offset[(size_t)p], src + (o * axis_len + s) * inner * (size_t)elem_size, bytes);
            offset[(size_t)p] += bytes;
            s += (size_t)parts[p];
        }
        if (s != axis_len) return ORC_ERR_ARG;
    }
    return ORC_OK;
}

int orc_where(const uint8_t *cond, int c_rank, const int64_t *c_dims, const float *x, int x_rank, const int64_t *x_dims,
              const float *y, int y_rank, const int64_t *y_dims, float *out, int strict, int *no_reference_kernel) {
    const bool same_cy = c_rank == y_rank && std::equal(c_dims, c_dims + c_rank, y_dims);
    const bool p1 = same_cy && orc_is_scalar(x_rank, x_dims);
    const bool p2 = orc_is_scalar(y_rank, y_dims) && x_rank == 4 && c_rank == 4 && c_dims[0] == 1 && c_dims[1] == 1;
    if (no_reference_kernel) *no_reference_kernel = (p1 || p2) ? 0 : 1;
    if (p1) {  // session.rs:947-956
        const size_t n = total_of(c_rank, c_dims);
        for (size_t i = 0; i < n; i++) out[i] = cond[i] ? x[0] : y[i];
        return ORC_OK;
    }
    if (p2 && c_dims[2] == x_dims[2] && c_dims[3] == x_dims[3]) {  // session.rs:958-987
        const size_t plane = (size_t)(x_dims[2] * x_dims[3]), planes = (size_t)(x_dims[0] * x_dims[1]);
        for (size_t p = 0; p < planes; p++)
            for (size_t i = 0; i < plane; i++) out[p * plane + i] = cond[i] ? x[p * plane + i] : y[0];
        return ORC_OK;
    }
    if (no_reference_kernel) *no_reference_kernel = 1;
    if (strict) return ORC_ERR_UNSUPPORTED;
    const int ranks[3] = {c_rank, x_rank, y_rank};
    const int64_t *shapes[3] = {c_dims, x_dims, y_dims};
    int out_rank = 0;
    int64_t out_dims[16], cs[16], xs[16], ys[16];
    if (orc_broadcast(3, ranks, shapes, &out_rank, out_dims)) return ORC_ERR_BROADCAST;
    if (orc_strides_for_broadcasting(c_rank, c_dims, out_rank, out_dims, cs) ||
        orc_strides_for_broadcasting(x_rank, x_dims, out_rank, out_dims, xs) ||
        orc_strides_for_broadcasting(y_rank, y_dims, out_rank, out_dims, ys))
        return ORC_ERR_BROADCAST;
    const size_t n = total_of(out_rank, out_dims);
    std::vector<int64_t> idx((size_t)out_rank, 0);
    for (size_t i = 0; i < n; i++) {
        int64_t ci = 0, xi = 0, yi = 0;
        for (int d = 0; d < out_rank; d++) {
            ci += idx[(size_t)d] * cs[d];
            xi += idx[(size_t)d] * xs[d];
            yi += idx[(size_t)d] * ys[d];
        }
        out[i] = cond[ci] ? x[xi] : y[yi];
        for (int d = out_rank - 1; d >= 0; d--) {
            if (++idx[(size_t)d] < out_dims[d]) break;
            idx[(size_t)d] = 0;
        }
    }
    return ORC_OK;
}

int orc_greater(const float *a, int a_rank, const int64_t *a_dims, const float *b, int b_rank, const int64_t *b_dims,
                uint8_t *out, int strict, int *no_reference_kernel) {
    const bool ref = orc_is_scalar(b_rank, b_dims) != 0;
    if (no_reference_kernel) *no_reference_kernel = ref ? 0 : 1;
    if (ref) {
        const size_t n = total_of(a_rank, a_dims);
        for (size_t i = 0; i < n; i++) out[i] = a[i] > b[0] ? 1 : 0;
        return ORC_OK;
    }
    if (strict) return ORC_ERR_UNSUPPORTED;
    const int ranks[2] = {a_rank, b_rank};
    const int64_t *shapes[2] = {a_dims, b_dims};
    int out_rank = 0;
    int64_t out_dims[16], as[16], bs[16];
    if (orc_broadcast(2, ranks, shapes, &out_rank, out_dims)) return ORC_ERR_BROADCAST;
    if (orc_strides_for_broadcasting(a_rank, a_dims, out_rank, out_dims, as) ||
        orc_strides_for_broadcasting(b_rank, b_dims, out_rank, out_dims, bs))
        return ORC_ERR_BROADCAST;
    const size_t n = total_of(out_rank, out_dims);
    std::vector<int64_t> idx((size_t)out_rank, 0);
    for (size_t i = 0; i < n; i++) {
        int64_t ai = 0, bi = 0;
        for (int d = 0; d < out_rank; d++) {
            ai += idx[(size_t)d] * as[d];
            bi += idx[(size_t)d] * bs[d];
        }
        out[i] = a[ai] > b[bi] ? 1 : 0;
        for (int d = out_rank - 1; d >= 0; d--) {
            if (++idx[(size_t)d] < out_dims[d]) break;
            idx[(size_t)d] = 0;
        }
    }
    return ORC_OK;
}

// Rust `as`: float -> int truncates toward zero, saturates, NaN -> 0; int -> narrower int wraps.
static int32_t f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
static int64_t f32_as_i64(float v) {
    if (v != v) return 0;
    if (v >= 9223372036854775808.0f) return INT64_MAX;
    if (v <= -9223372036854775808.0f) return INT64_MIN;
    return (int64_t)v;
}

int orc_cast(const void *in, int from, void *out, int to, size_t n, int strict, int *no_reference_kernel) {
    enum { B = 0, F = 1, I4 = 2, I8 = 3 };
    const bool ref = (from == I4 && to == F) || (from == I8 && to == I4) || (from == I8 && to == F) || (from == F && to == B);
    if (no_reference_kernel) *no_reference_kernel = ref ? 0 : 1;
    if (!ref && strict) return ORC_ERR_UNSUPPORTED;
    for (size_t i = 0; i < n; i++) {
        int64_t iv = 0;
        float fv = 0;
        switch (from) {
        case B: iv = static_cast<const uint8_t *>(in)[i] ? 1 : 0; fv = (float)iv; break;
        case F: fv = static_cast<const float *>(in)[i]; break;
        case I4: iv = static_cast<const int32_t *>(in)[i]; fv = (float)iv; break;
        case I8: iv = static_cast<const int64_t *>(in)[i]; fv = (float)iv; break;
        default: return ORC_ERR_ARG;
        }
        switch (to) {
        case B: static_cast<uint8_t *>(out)[i] = from == F ? (fv != 0.0f) : (iv != 0); break;
        case F: static_cast<float *>(out)[i] = fv; break;
        case I4: static_cast<int32_t *>(out)[i] = from == F ? f32_as_i32(fv) : (int32_t)(uint32_t)(uint64_t)iv; break;
        case I8: static_cast<int64_t *>(out)[i] = from == F ? f32_as_i64(fv) : iv; break;
        default: return ORC_ERR_ARG;
        }
    }
    return ORC_OK;
}

int orc_batchnorm(const float *x, const float *scale, const float *bias, const float *mean, const float *var, float *out,
                  size_t n, size_t c, size_t h, size_t w, float eps) {
    for (size_t in_ = 0; in_ < n; in_++)
        for (size_t ch = 0; ch < c; ch++)
            for (size_t i = 0; i < h * w; i++) {
                const size_t off = (in_ * c + ch) * h * w + i;
                out[off] = ((x[off] - mean[ch]) / std::sqrt(var[ch] + eps)) * scale[ch] + bias[ch];
            }
    return ORC_OK;
}

int orc_global_average_pool(const float *x, float *out, size_t n, size_t c, size_t h, size_t w) {
    const size_t area = h * w;
    for (size_t p = 0; p < n * c; p++) {
        float sum = 0.0f;  // Iterator::sum::<f32>() folds from 0.0 in order
        for (size_t i = 0; i < area; i++) sum += x[p * area + i];
        out[p] = sum / (float)area;
    }
    return ORC_OK;
}

int orc_leaky_relu(const float *x, float *out, size_t n, float alpha) {
    for (size_t i = 0; i < n; i++) out[i] = x[i] < 0.0f ? alpha * x[i] : x[i];
    return ORC_OK;
}

int orc_sgemm(int trans_a, int trans_b, size_t m, size_t k, size_t n, float alpha, const float *a, size_t lda,
              const float *b, size_t ldb, float beta, float *c, size_t ldc) {
    const size_t KC = 256;
    if (k == 0) {
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) c[i * ldc + j] = beta == 0.0f ? 0.0f : beta * c[i * ldc + j];
        return ORC_OK;
    }
    for (size_t k0 = 0; k0 < k; k0 += KC) {
        const size_t k1 = std::min(k, k0 + KC);
        const float bt = k0 == 0 ? beta : 1.0f;
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) {
                float ab = 0.0f;
                for (size_t p = k0; p < k1; p++) {
                    const float av = trans_a ? a[p * lda + i] : a[i * lda + p];
                    const float bv = trans_b ? b[j * ldb + p] : b[p * ldb + j];
                    ab = std::fma(av, bv, ab);
                }
                float &cv = c[i * ldc + j];
                cv = bt == 0.0f ? alpha * ab : bt * cv + alpha * ab;
            }
    }
    return ORC_OK;
}

int orc_conv2d(const float *x, const float *w, const float *bias, float *out, size_t batch, size_t c, size_t ih, size_t iw,
               size_t oc, size_t oh, size_t ow, size_t kh, size_t kw, size_t sh, size_t sw, size_t dh, size_t dw, size_t pad_t,
               size_t pad_l, size_t group) {
    if (group == 0 || c % group || oc % group) return ORC_ERR_ARG;
    const size_t ohw = oh * ow, cg = c / group, ocg = oc / group, k = cg * kh * kw;
    for (size_t b = 0; b < batch; b++)  // conv2d.rs:63-80
        for (size_t o = 0; o < oc; o++)
            for (size_t i = 0; i < ohw; i++) out[(b * oc + o) * ohw + i] = bias ? bias[o] : 0.0f;
    std::vector<float> col(batch * c * kh * kw * ohw);
    for (size_t b = 0; b < batch; b++)
        for (size_t ch = 0; ch < c; ch++)
            for (size_t fy = 0; fy < kh; fy++)
                for (size_t fx = 0; fx < kw; fx++)
                    for (size_t y = 0; y < oh; y++)
                        for (size_t xo = 0; xo < ow; xo++) {
                            const long iy = (long)(y * sh + fy * dh) - (long)pad_t, ix = (long)(xo * sw + fx * dw) - (long)pad_l;
                            const bool in = iy >= 0 && iy < (long)ih && ix >= 0 && ix < (long)iw;
                            col[((((b * c + ch) * kh + fy) * kw + fx) * oh + y) * ow + xo] =
                                in ? x[((b * c + ch) * ih + (size_t)iy) * iw + (size_t)ix] : 0.0f;
                        }
    // conv2d.rs:152-210: chunks of col (per image and group) against the weights of the group, cycling.
    for (size_t b = 0; b < batch; b++)
        for (size_t g = 0; g < group; g++)
            orc_sgemm(0, 0, ocg, k, ohw, 1.0f, w + g * ocg * k, k, col.data() + (b * group + g) * k * ohw, ohw, 1.0f,
                      out + (b * group + g) * ocg * ohw, ohw);
    return ORC_OK;
}

int orc_max_pool(const float *x, float *out, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow, size_t kh, size_t kw,
                 size_t sh, size_t sw, size_t pad_t, size_t pad_l) {
    const float lowest = -3.40282347e+38f;
    for (size_t p = 0; p < planes; p++)
        for (size_t ay = 0; ay < oh; ay++)
            for (size_t ax = 0; ax < ow; ax++) {
                const long y = (long)(ay * sh) - (long)pad_t, xx = (long)(ax * sw) - (long)pad_l;
                float m = lowest;
                for (size_t fy = 0; fy < kh; fy++)
                    for (size_t fx = 0; fx < kw; fx++) {
                        const long oy = y + (long)fy, ox = xx + (long)fx;
                        if (oy < 0 || oy >= (long)ih || ox < 0 || ox >= (long)iw) continue;
                        const float v = x[(p * ih + (size_t)oy) * iw + (size_t)ox];
                        m = std::fmax(v, m);  // f32::max: NaN loses
                    }
                out[(p * oh + ay) * ow + ax] = m == lowest ? 0.0f : m;
            }
    return ORC_OK;
}

int orc_resize(const float *x, float *out, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow, int nearest) {
    if (ih == 0 || iw == 0) return ORC_ERR_ARG;
    const float sh = (float)oh / (float)ih, sw = (float)ow / (float)iw;
    for (size_t p = 0; p < planes; p++) {
        const float *in = x + p * ih * iw;
        float *o = out + p * oh * ow;
        for (size_t h = 0; h < oh; h++)
            for (size_t w = 0; w < ow; w++) {
                if (nearest) {  // session.rs:1078-1090
                    size_t y = (size_t)((float)h / sh), xx = (size_t)((float)w / sw);
                    y = std::min(y, ih - 1);
                    xx = std::min(xx, iw - 1);
                    o[h * ow + w] = in[y * iw + xx];
                } else {  // session.rs:1099-1121
                    const float ihf = std::fmax((float)h / sh - 0.5f, 0.0f), iwf = std::fmax((float)w / sw - 0.5f, 0.0f);
                    const size_t y = (size_t)ihf, xx = (size_t)iwf;
                    const size_t y0 = std::min(y, ih - 1), y1 = std::min(y + 1, ih - 1);
                    const size_t x0 = std::min(xx, iw - 1), x1 = std::min(xx + 1, iw - 1);
                    const float v00 = in[y0 * iw + x0], v01 = in[y0 * iw + x1], v10 = in[y1 * iw + x0], v11 = in[y1 * iw + x1];
                    const float hd = v00 + (v10 - v00) * (ihf - (float)y);
                    const float hw = v01 + (v11 - v01) * (ihf - (float)y);
                    o[h * ow + w] = hd + (hw - hd) * (iwf - (float)xx);
                }
            }
    }
    return ORC_OK;
}

float orc_fast_sum(const float *x, size_t n) { return fast_sum(x, n); }
float orc_fast_sum_squares(const float *x, size_t n) { return fast_sum_squares(x, n); }
void orc_faster_pow2(const float *p, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = faster_pow2(p[i]);
}

}  // extern "C"
