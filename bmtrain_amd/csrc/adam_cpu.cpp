// Host-memory Adam step (optimizer offload) and the fp32 -> 16-bit host converters.
// Replaces csrc/include/adam_cpu.hpp:139-175 and :183-557 of the reference.
//
// This file is compiled with -ffp-contract=off: the only fused multiply-adds are
// the explicit ones, so results do not depend on the compiler.  Two expression
// trees exist, as in the reference's compiled code, and which elements take which
// is reproduced exactly so that results are bit-identical to it for the same SIMD
// level and thread count:
//   * "wide" tree (fp16 gradients, whole SIMD groups of a thread's chunk;
//     adam_cpu.hpp:353-382, :454-486):
//       g = g16/scale; m' = fma(b1,m,(1-b1)*g); v' = fma(b2,v,(1-b2)*(g*g));
//       p1 = fma(-lr, wd*p, p); p' = fma(-lr, (m'/bc1)/(sqrt(v'/bc2)+eps), p1)
//   * "narrow" tree (fp16 chunk remainders, every bf16 element; adam_cpu.hpp:207-218,
//     :265-276 as contracted by the reference's host compiler):
//       m' = fma(b1,m,(1-b1)*g); v' = fma(b2,v,((1-b2)*g)*g);
//       p' = fma(-(lr*wd), p, p - ((lr*m')/bc1)/(sqrt(v'/bc2)+eps))
// Both trees are evaluated here with 16-lane AVX-512 or 8-lane AVX2 instructions when
// the CPU has them (every operation is IEEE-exact per lane, so vector and scalar code
// agree bit for bit); the bf16 path, scalar in the reference, is vectorised as well.
// Work is split over one thread per CPU of the calling thread's affinity mask, in
// contiguous chunks of ceil(n / threads) elements (adam_cpu.hpp:42-80); the threads are kept
// between calls instead of being created and joined every time.
#include "../../include/bmt_hip.h"

#include <immintrin.h>
#include <sched.h>

#include <pthread.h>

#include <algorithm>
#include <cmath>
#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

namespace bmt {
int fail_message(int code, const char *what);  // host.cpp
}

namespace {

struct Hyper {
    float b1, b2, eps, lr, scale, wd, bc1, bc2;
};

// ---- scalar converters -----------------------------------------------------------
inline uint32_t bits_of(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float float_of(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, em = h & 0x7FFFu;
    if (em >= 0x7C00u) return float_of(sign | 0x7F800000u | ((em & 0x3FFu) << 13));
    if (em < 0x0400u) return float_of(bits_of((float)em * 0x1p-24f) | sign);
    return float_of(sign | ((em << 13) + 0x38000000u));
}
inline uint16_t float_to_half(float f) {  // round to nearest even
    const uint32_t u = bits_of(f), a = u & 0x7FFFFFFFu;
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    if (a > 0x7F800000u) return sign | 0x7E00u;
    if (a >= 0x47800000u) return sign | 0x7C00u;
    if (a < 0x38800000u) {
        // Adding 0.5 places the value's 2^-24 digit at the float's last mantissa bit, so the
        // addition itself performs the round-to-nearest-even; the low bits then hold the result.
        const float r = float_of(a) + 0.5f;
        return sign | (uint16_t)(bits_of(r) - 0x3F000000u);
    }
    const uint32_t r = a - 0x38000000u;
    return sign | (uint16_t)((r + 0x0FFFu + ((r >> 13) & 1u)) >> 13);
}
inline float bf16_to_float(uint16_t h) { return float_of((uint32_t)h << 16); }
inline uint16_t float_to_bf16_trunc(float f) { return (uint16_t)(bits_of(f) >> 16); }

// ---- one element, scalar ------------------------------------------------------------
struct Delta { float sum = 0.f, sumsq = 0.f; };

inline void narrow_elem(float g, float &m, float &v, float &p, const Hyper &h, Delta *d) {
    const float mm = std::fmaf(h.b1, m, (1.0f - h.b1) * g);
    const float vv = std::fmaf(h.b2, v, ((1.0f - h.b2) * g) * g);
    const float den = std::sqrt(vv / h.bc2) + h.eps;
    if (d) { const float x = (mm / h.bc1) / den + h.wd * p; d->sum += x; d->sumsq += x * x; }
    const float upd = ((h.lr * mm) / h.bc1) / den;
    const float np = std::fmaf(-(h.lr * h.wd), p, p - upd);
    m = mm; v = vv; p = np;
}

// ---- 16-lane bodies -------------------------------------------------------------------
#define BMT_AVX512 __attribute__((target("avx512f,f16c,fma")))
#define BMT_AVX2 __attribute__((target("avx,f16c,fma")))

BMT_AVX512 inline void delta_acc16(__m512 x, Delta *d) {
    alignas(64) float t[16];
    _mm512_store_ps(t, x);
    for (int k = 0; k < 16; k++) { d->sum += t[k]; d->sumsq += t[k] * t[k]; }
}

// fp16 gradients, wide tree on whole groups of 16, narrow tree on the remainder.
BMT_AVX512 void fp16_chunk_avx512(int64_t lo, int64_t hi, float *p32, uint16_t *p16, const uint16_t *g16, float *mo,
                                  float *va, const Hyper &h, Delta *d) {
    const __m512 b1 = _mm512_set1_ps(h.b1), b2 = _mm512_set1_ps(h.b2), c1 = _mm512_set1_ps(1.0f - h.b1),
                 c2 = _mm512_set1_ps(1.0f - h.b2), eps = _mm512_set1_ps(h.eps), nlr = _mm512_set1_ps(-h.lr),
                 sc = _mm512_set1_ps(h.scale), wd = _mm512_set1_ps(h.wd), bc1 = _mm512_set1_ps(h.bc1),
                 bc2 = _mm512_set1_ps(h.bc2);
    int64_t j = lo;
    for (; j + 16 <= hi; j += 16) {
        const __m512 g = _mm512_div_ps(_mm512_cvtph_ps(_mm256_loadu_si256((const __m256i *)(g16 + j))), sc);
        __m512 m = _mm512_loadu_ps(mo + j), v = _mm512_loadu_ps(va + j), p = _mm512_loadu_ps(p32 + j);
        m = _mm512_fmadd_ps(b1, m, _mm512_mul_ps(c1, g));
        v = _mm512_fmadd_ps(b2, v, _mm512_mul_ps(c2, _mm512_mul_ps(g, g)));
        const __m512 q = _mm512_div_ps(_mm512_div_ps(m, bc1), _mm512_add_ps(_mm512_sqrt_ps(_mm512_div_ps(v, bc2)), eps));
        if (d) delta_acc16(_mm512_add_ps(q, _mm512_mul_ps(wd, p)), d);
        p = _mm512_fmadd_ps(nlr, _mm512_mul_ps(wd, p), p);
        p = _mm512_fmadd_ps(nlr, q, p);
        _mm512_storeu_ps(p32 + j, p);
        _mm256_storeu_si256((__m256i *)(p16 + j), _mm512_cvtps_ph(p, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        _mm512_storeu_ps(mo + j, m);
        _mm512_storeu_ps(va + j, v);
    }
    for (; j < hi; j++) {
        narrow_elem(half_to_float(g16[j]) / h.scale, mo[j], va[j], p32[j], h, d);
        p16[j] = float_to_half(p32[j]);
    }
}

// bf16 gradients: narrow tree everywhere, 16 lanes at a time.
BMT_AVX512 void bf16_chunk_avx512(int64_t lo, int64_t hi, float *p32, uint16_t *p16, const uint16_t *g16, float *mo,
                                  float *va, const Hyper &h, Delta *d) {
    const __m512 b1 = _mm512_set1_ps(h.b1), b2 = _mm512_set1_ps(h.b2), c1 = _mm512_set1_ps(1.0f - h.b1),
                 c2 = _mm512_set1_ps(1.0f - h.b2), eps = _mm512_set1_ps(h.eps), lr = _mm512_set1_ps(h.lr),
                 sc = _mm512_set1_ps(h.scale), wd = _mm512_set1_ps(h.wd), bc1 = _mm512_set1_ps(h.bc1),
                 bc2 = _mm512_set1_ps(h.bc2), nlrwd = _mm512_set1_ps(-(h.lr * h.wd));
    int64_t j = lo;
    for (; j + 16 <= hi; j += 16) {
        const __m512i gi = _mm512_slli_epi32(_mm512_cvtepu16_epi32(_mm256_loadu_si256((const __m256i *)(g16 + j))), 16);
        const __m512 g = _mm512_div_ps(_mm512_castsi512_ps(gi), sc);
        __m512 m = _mm512_loadu_ps(mo + j), v = _mm512_loadu_ps(va + j), p = _mm512_loadu_ps(p32 + j);
        m = _mm512_fmadd_ps(b1, m, _mm512_mul_ps(c1, g));
        v = _mm512_fmadd_ps(b2, v, _mm512_mul_ps(_mm512_mul_ps(c2, g), g));
        const __m512 den = _mm512_add_ps(_mm512_sqrt_ps(_mm512_div_ps(v, bc2)), eps);
        if (d) delta_acc16(_mm512_add_ps(_mm512_div_ps(_mm512_div_ps(m, bc1), den), _mm512_mul_ps(wd, p)), d);
        const __m512 upd = _mm512_div_ps(_mm512_div_ps(_mm512_mul_ps(lr, m), bc1), den);
        p = _mm512_fmadd_ps(nlrwd, p, _mm512_sub_ps(p, upd));
        _mm512_storeu_ps(p32 + j, p);
        _mm256_storeu_si256((__m256i *)(p16 + j), _mm512_cvtepi32_epi16(_mm512_srli_epi32(_mm512_castps_si512(p), 16)));
        _mm512_storeu_ps(mo + j, m);
        _mm512_storeu_ps(va + j, v);
    }
    for (; j < hi; j++) {
        narrow_elem(bf16_to_float(g16[j]) / h.scale, mo[j], va[j], p32[j], h, d);
        p16[j] = float_to_bf16_trunc(p32[j]);
    }
}

// ---- 8-lane bodies --------------------------------------------------------------------
BMT_AVX2 inline void delta_acc8(__m256 x, Delta *d) {
    alignas(32) float t[8];
    _mm256_store_ps(t, x);
    for (int k = 0; k < 8; k++) { d->sum += t[k]; d->sumsq += t[k] * t[k]; }
}

BMT_AVX2 void fp16_chunk_avx2(int64_t lo, int64_t hi, float *p32, uint16_t *p16, const uint16_t *g16, float *mo,
                              float *va, const Hyper &h, Delta *d) {
    const __m256 b1 = _mm256_set1_ps(h.b1), b2 = _mm256_set1_ps(h.b2), c1 = _mm256_set1_ps(1.0f - h.b1),
                 c2 = _mm256_set1_ps(1.0f - h.b2), eps = _mm256_set1_ps(h.eps), nlr = _mm256_set1_ps(-h.lr),
                 sc = _mm256_set1_ps(h.scale), wd = _mm256_set1_ps(h.wd), bc1 = _mm256_set1_ps(h.bc1),
                 bc2 = _mm256_set1_ps(h.bc2);
    int64_t j = lo;
    for (; j + 8 <= hi; j += 8) {
        const __m256 g = _mm256_div_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(g16 + j))), sc);
        __m256 m = _mm256_loadu_ps(mo + j), v = _mm256_loadu_ps(va + j), p = _mm256_loadu_ps(p32 + j);
        m = _mm256_fmadd_ps(b1, m, _mm256_mul_ps(c1, g));
        v = _mm256_fmadd_ps(b2, v, _mm256_mul_ps(c2, _mm256_mul_ps(g, g)));
        const __m256 q = _mm256_div_ps(_mm256_div_ps(m, bc1), _mm256_add_ps(_mm256_sqrt_ps(_mm256_div_ps(v, bc2)), eps));
        if (d) delta_acc8(_mm256_add_ps(q, _mm256_mul_ps(wd, p)), d);
        p = _mm256_fmadd_ps(nlr, _mm256_mul_ps(wd, p), p);
        p = _mm256_fmadd_ps(nlr, q, p);
        _mm256_storeu_ps(p32 + j, p);
        _mm_storeu_si128((__m128i *)(p16 + j), _mm256_cvtps_ph(p, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        _mm256_storeu_ps(mo + j, m);
        _mm256_storeu_ps(va + j, v);
    }
    for (; j < hi; j++) {
        narrow_elem(half_to_float(g16[j]) / h.scale, mo[j], va[j], p32[j], h, d);
        p16[j] = float_to_half(p32[j]);
    }
}

// ---- scalar bodies ----------------------------------------------------------------------
void fp16_chunk_scalar(int64_t lo, int64_t hi, float *p32, uint16_t *p16, const uint16_t *g16, float *mo, float *va,
                       const Hyper &h, Delta *d) {
    for (int64_t j = lo; j < hi; j++) {
        narrow_elem(half_to_float(g16[j]) / h.scale, mo[j], va[j], p32[j], h, d);
        p16[j] = float_to_half(p32[j]);
    }
}
void bf16_chunk_scalar(int64_t lo, int64_t hi, float *p32, uint16_t *p16, const uint16_t *g16, float *mo, float *va,
                       const Hyper &h, Delta *d) {
    for (int64_t j = lo; j < hi; j++) {
        narrow_elem(bf16_to_float(g16[j]) / h.scale, mo[j], va[j], p32[j], h, d);
        p16[j] = float_to_bf16_trunc(p32[j]);
    }
}

// SIMD level in the reference's terms (cpu_info.h:7-38): 2 = AVX-512F, 1 = AVX+FMA+F16C, 0 = neither.
int simd_level() {
    static const int level = [] {
        __builtin_cpu_init();
        const bool narrow = __builtin_cpu_supports("avx") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c");
        if (__builtin_cpu_supports("avx512f") && narrow) return 2;
        if (narrow) return 1;
        return 0;
    }();
    return level;
}

int affinity_cpus() {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof(set), &set) != 0) return 1;
    const int n = CPU_COUNT(&set);
    return n > 0 ? n : 1;
}

// ---- worker threads ------------------------------------------------------------------------
// The reference creates and joins one std::thread per chunk on every call (adam_cpu.hpp:61-75).
// Here the helpers are created once and parked on a condition variable; the calling thread takes
// chunk 0 itself.  The pool is rebuilt when the affinity mask asks for a different thread count
// and is abandoned (not joined) in a forked child and at process exit, where its threads either
// do not exist or are parked.
class WorkerPool {
public:
    explicit WorkerPool(int helpers) {
        for (int i = 0; i < helpers; i++) threads_.emplace_back([this, i] { loop(i + 1); });
    }
    ~WorkerPool() {
        {
            std::lock_guard<std::mutex> lock(mu_);
            stop_ = true;
            generation_.fetch_add(1, std::memory_order_release);
        }
        wake_.notify_all();
        for (auto &t : threads_) t.join();
    }
    int helpers() const { return (int)threads_.size(); }

    // Runs job(slot) for slot = 0 .. helpers(); returns when all have finished.
    void run(const std::function<void(int)> &job) {
        {
            std::lock_guard<std::mutex> lock(mu_);
            job_ = &job;
            pending_.store((int)threads_.size(), std::memory_order_relaxed);
            generation_.fetch_add(1, std::memory_order_release);
        }
        wake_.notify_all();
        job(0);
        for (int spin = 0; spin < kSpinPolls && pending_.load(std::memory_order_acquire) != 0; spin++)
            __builtin_ia32_pause();
        std::unique_lock<std::mutex> lock(mu_);
        done_.wait(lock, [this] { return pending_.load(std::memory_order_relaxed) == 0; });
        job_ = nullptr;
    }

private:
    void loop(int slot) {
        uint64_t seen = 0;
        for (;;) {
            const std::function<void(int)> *job = nullptr;
            // Calls often come in quick succession (one per piece of a tensor that is being copied in):
            // poll for the next job for a short while before going to sleep on the condition variable.
            for (int spin = 0; spin < kSpinPolls && generation_.load(std::memory_order_acquire) == seen; spin++)
                __builtin_ia32_pause();
            {
                std::unique_lock<std::mutex> lock(mu_);
                wake_.wait(lock, [&] { return generation_.load(std::memory_order_relaxed) != seen; });
                seen = generation_.load(std::memory_order_relaxed);
                if (stop_) return;
                job = job_;
            }
            (*job)(slot);
            {
                std::lock_guard<std::mutex> lock(mu_);
                if (pending_.fetch_sub(1, std::memory_order_acq_rel) == 1) done_.notify_one();
            }
        }
    }

    std::vector<std::thread> threads_;
    std::mutex mu_;
    std::condition_variable wake_, done_;
    const std::function<void(int)> *job_ = nullptr;
    // Roughly a millisecond of polling before a thread goes to sleep.  It buys back-to-back calls a start on all
    // cores at once; under a CPU quota smaller than the affinity mask it costs that millisecond per call
    // (BMT_HOST_ADAM_SPIN=0 in the environment turns the polling off).
    static inline const int kSpinPolls = [] {
        const char *e = getenv("BMT_HOST_ADAM_SPIN");
        return e ? atoi(e) : 200000;
    }();
    std::atomic<uint64_t> generation_{0};
    std::atomic<int> pending_{0};
    bool stop_ = false;
};

std::mutex g_pool_mutex;           // one fan-out at a time
WorkerPool *g_pool = nullptr;      // leaked on purpose at exit
void forget_pool_in_child() { g_pool = nullptr; new (&g_pool_mutex) std::mutex(); }

// Runs body(lo, hi, slot) over [0, n) split into `threads` contiguous chunks of
// ceil(n / threads) elements (threads = CPUs in the caller's affinity mask, adam_cpu.hpp:54-58);
// slot t is private to chunk t.  The caller reads the thread count (once per call: the mask can change under
// a running process) and sizes whatever it indexes by slot from the same value.
template <typename Body>
void fan_out(int64_t n, int64_t threads, const Body &body) {
    const int64_t chunk = std::max<int64_t>((n + threads - 1) / threads, 1);
    if (threads == 1) { body(0, n, 0); return; }
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    static const bool registered = (pthread_atfork(nullptr, nullptr, forget_pool_in_child), true);
    (void)registered;
    if (g_pool == nullptr || g_pool->helpers() != (int)threads - 1) {
        delete g_pool;
        g_pool = new WorkerPool((int)threads - 1);
    }
    const std::function<void(int)> job = [&](int t) {
        const int64_t lo = std::min((int64_t)t * chunk, n), hi = std::min((int64_t)(t + 1) * chunk, n);
        if (lo < hi) body(lo, hi, t);
    };
    g_pool->run(job);
}

using ChunkFn = void (*)(int64_t, int64_t, float *, uint16_t *, const uint16_t *, float *, float *, const Hyper &, Delta *);

int run(ChunkFn fn, int64_t n, void *p32, void *p16, void *delta_info, const void *g16, void *m, void *v, const Hyper &h) {
    if (n <= 0) return 0;
    if (!p32 || !p16 || !g16 || !m || !v) return bmt::fail_message(-1, "adam_cpu launcher: null pointer");
    const int64_t threads = affinity_cpus();
    std::vector<Delta> parts((size_t)threads);
    fan_out(n, threads, [&](int64_t lo, int64_t hi, int slot) {
        fn(lo, hi, (float *)p32, (uint16_t *)p16, (const uint16_t *)g16, (float *)m, (float *)v, h,
           delta_info ? &parts[(size_t)slot] : nullptr);
    });
    if (delta_info) {
        float sum = 0.f, sumsq = 0.f;
        for (const Delta &d : parts) { sum += d.sum; sumsq += d.sumsq; }
        float *out = (float *)delta_info;
        out[0] = sum / n;                                   // adam_cpu.hpp:233-238
        out[1] = sumsq / n - sum * sum / ((float)n * (float)n);
        out[2] = sum;
        out[3] = sumsq;
    }
    return 0;
}

}  // namespace

extern "C" int adam_cpu_fp16_launcher(int64_t n, void *param_fp32, void *param_fp16, void *delta_info, const void *g_fp16,
                                      void *m_fp32, void *v_fp32, float beta1, float beta2, float eps, float lr,
                                      float scale, float weight_decay, float bias_correction1, float bias_correction2) {
    const Hyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    const int level = simd_level();
    ChunkFn fn = level == 2 ? fp16_chunk_avx512 : (level == 1 ? fp16_chunk_avx2 : fp16_chunk_scalar);
    return run(fn, n, param_fp32, param_fp16, delta_info, g_fp16, m_fp32, v_fp32, h);
}

extern "C" int adam_cpu_bf16_launcher(int64_t n, void *param_fp32, void *param_bf16, void *delta_info, const void *g_bf16,
                                      void *m_fp32, void *v_fp32, float beta1, float beta2, float eps, float lr,
                                      float scale, float weight_decay, float bias_correction1, float bias_correction2) {
    const Hyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    ChunkFn fn = simd_level() == 2 ? bf16_chunk_avx512 : bf16_chunk_scalar;
    return run(fn, n, param_fp32, param_bf16, delta_info, g_bf16, m_fp32, v_fp32, h);
}

extern "C" int to_fp16_from_fp32(int64_t n, const void *param_fp32, void *param_fp16) {
    if (n <= 0) return 0;
    if (!param_fp32 || !param_fp16) return bmt::fail_message(-1, "to_fp16_from_fp32: null pointer");
    const float *src = (const float *)param_fp32;
    uint16_t *dst = (uint16_t *)param_fp16;
    fan_out(n, affinity_cpus(), [=](int64_t lo, int64_t hi, int) { for (int64_t i = lo; i < hi; i++) dst[i] = float_to_half(src[i]); });
    return 0;
}

extern "C" int to_bf16_from_fp32(int64_t n, const void *param_fp32, void *param_bf16) {
    if (n <= 0) return 0;
    if (!param_fp32 || !param_bf16) return bmt::fail_message(-1, "to_bf16_from_fp32: null pointer");
    const float *src = (const float *)param_fp32;
    uint16_t *dst = (uint16_t *)param_bf16;
    fan_out(n, affinity_cpus(), [=](int64_t lo, int64_t hi, int) { for (int64_t i = lo; i < hi; i++) dst[i] = float_to_bf16_trunc(src[i]); });
    return 0;
}
