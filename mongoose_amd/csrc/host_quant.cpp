// host_quant.cpp -- host-side weight preparation for the HIP backend: the Q8
// per-row quantizer the reference runs in Go before upload, the GGML Q4_0
// block quantizer, fp16 conversion, the split-layout repack for Q4_0 rows and a
// machine-independent synthetic weight generator.  No device code.
#pragma STDC FP_CONTRACT OFF
#include "../../include/mongoose_hip.h"
#include "host_util.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace mg {

// A fixed set of worker threads shared by every host-side loop of the library (starting threads per
// loop costs more than the per-layer staging loops themselves).  One parallel region at a time; the
// calling thread takes jobs too.  Jobs must not start a region themselves.
class WorkPool {
    // Each parallel region has its own state object: a worker that wakes late holds the region it was
    // woken for, finds its job counter exhausted and never touches a later region's function.
    struct Region {
        const std::function<void(size_t)>* fn;
        size_t total;
        std::atomic<size_t> next{0};
        std::atomic<size_t> remaining;
    };

public:
    static WorkPool& get() {
        static WorkPool* pool = new WorkPool();      // lives until the process ends
        return *pool;
    }
    void run(size_t njobs, const std::function<void(size_t)>& fn) {
        if (njobs == 0) return;
        if (njobs == 1 || nWorkers == 0) {
            for (size_t j = 0; j < njobs; j++) fn(j);
            return;
        }
        std::lock_guard<std::mutex> region(regionMutex);
        auto r = std::make_shared<Region>();
        r->fn = &fn; r->total = njobs; r->remaining.store(njobs);
        {
            std::lock_guard<std::mutex> lk(m);
            current = r;
            generation++;
        }
        wake.notify_all();
        work(*r);
        std::unique_lock<std::mutex> lk(m);
        done.wait(lk, [&] { return r->remaining.load() == 0; });
    }

private:
    WorkPool() {
        unsigned hw = std::thread::hardware_concurrency();
        if (hw == 0) hw = 1;
        if (hw > 16) hw = 16;
        nWorkers = hw - 1;
        for (unsigned t = 0; t < nWorkers; t++) std::thread([this] { loop(); }).detach();
    }
    void work(Region& r) {
        for (;;) {
            const size_t j = r.next.fetch_add(1);
            if (j >= r.total) break;
            (*r.fn)(j);
            if (r.remaining.fetch_sub(1) == 1) {
                std::lock_guard<std::mutex> lk(m);
                done.notify_all();
            }
        }
    }
    void loop() {
        unsigned long seen = 0;
        for (;;) {
            std::shared_ptr<Region> r;
            {
                std::unique_lock<std::mutex> lk(m);
                wake.wait(lk, [&] { return generation != seen; });
                seen = generation;
                r = current;
            }
            if (r) work(*r);
        }
    }
    unsigned nWorkers = 0;
    std::mutex regionMutex, m;
    std::condition_variable wake, done;
    std::shared_ptr<Region> current;
    unsigned long generation = 0;
};

void parallel_jobs(size_t njobs, const std::function<void(size_t)>& fn) { WorkPool::get().run(njobs, fn); }

void parallel_for(size_t n, size_t grain, const std::function<void(size_t, size_t)>& fn) {
    if (n == 0) return;
    if (grain == 0) grain = 1;
    const size_t chunks = (n + grain - 1) / grain;
    if (chunks <= 1) { fn(0, n); return; }
    parallel_jobs(chunks, [&](size_t c) { fn(c * grain, std::min(n, (c + 1) * grain)); });
}

// Split layout read by the fast Q4_0 kernel: all 16-byte nibble groups of the
// matrix (row-major), then all fp16 block scales.  Same bytes as GGUF, only
// regrouped so that both are reachable with aligned loads.
void repack_q4_0_blocks(const uint8_t* raw, size_t nb, size_t b0, size_t b1, uint8_t* planar) {
    uint8_t* qs = planar;
    uint8_t* d = planar + nb * 16;
    for (size_t i = b0; i < b1; i++) {
        std::memcpy(qs + i * 16, raw + i * 18 + 2, 16);
        std::memcpy(d + i * 2, raw + i * 18, 2);
    }
}

void repack_q4_0_host(const uint8_t* raw, int rows, int cols, uint8_t* planar) {
    const size_t nb = (size_t)rows * (cols / 32);
    parallel_for(nb, 1 << 13, [&](size_t a, size_t b) { repack_q4_0_blocks(raw, nb, a, b, planar); });
}

}  // namespace mg

extern "C" {

// IEEE binary16 <-> binary32, round to nearest even (what GGML's
// GGML_FP32_TO_FP16 does; not the truncating helper of conductor.go:27-35).
uint16_t mg_f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x1ffu));   // NaN, payload kept
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                          // overflow -> inf
    if (x < 0x33000001u) return (uint16_t)sign;                                       // <= 2^-25 -> 0 (tie to even)
    uint32_t mant, shift, expBits;
    if (x < 0x38800000u) {            // subnormal half
        mant = (x & 0x7fffffu) | 0x800000u;
        shift = 126u - (x >> 23);
        expBits = 0;
    } else {
        mant = x & 0x7fffffu;
        shift = 13;
        expBits = ((x >> 23) - 112u) << 10;
    }
    uint32_t keep = mant >> shift;
    uint32_t dropped = mant & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    uint32_t r = expBits + keep;                     // '+' so a mantissa carry bumps the exponent
    if (dropped > halfway || (dropped == halfway && (keep & 1u))) r++;
    return (uint16_t)(sign | r);
}

float mg_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, x;
    if (e == 31) x = sign | 0x7f800000u | (m << 13);
    else if (e != 0) x = sign | ((e + 112u) << 23) | (m << 13);
    else if (m == 0) x = sign;
    else {
        // value = m * 2^-24; normalise
        int lz = __builtin_clz(m) - 21;              // shifts needed to bring bit 10 up
        m = (m << lz) & 0x3ffu;
        x = sign | ((uint32_t)(113 - lz) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// quantizeQ8, cuda_fused_infer.go:363-390 (mode 0), or the Metal loader's
// rounding, metal_impl_darwin.m:5765-5780 (mode 1).  scale = absmax/127.
void mg_quantize_q8(const float* w, int rows, int cols, int mode, int8_t* q, float* scales) {
    mg::parallel_for((size_t)rows, 16, [&](size_t r0, size_t r1) {
        for (size_t r = r0; r < r1; r++) {
            const float* src = w + r * (size_t)cols;
            int8_t* dst = q + r * (size_t)cols;
            float amax = 0.0f;
            for (int c = 0; c < cols; c++) {
                float v = std::fabs(src[c]);
                if (v > amax) amax = v;
            }
            const float s = amax / 127.0f;
            scales[r] = s;
            if (!(s > 0.0f)) { std::memset(dst, 0, (size_t)cols); continue; }
            if (mode == 0) {
                const float inv = 1.0f / s;
                for (int c = 0; c < cols; c++) {
                    const float t = src[c] * inv;
                    // Go's int(): truncate; NaN/overflow (only when 1/s overflowed) -> most negative
                    const bool inRange = t > -9.2233720368547758e18f && t < 9.2233720368547758e18f;
                    const long long v = inRange ? (long long)t : (-9223372036854775807LL - 1);
                    dst[c] = (int8_t)std::min(127LL, std::max(-128LL, v));
                }
            } else {
                const float inv = 127.0f / amax;
                for (int c = 0; c < cols; c++) {
                    float v = std::min(127.0f, std::max(-127.0f, src[c] * inv));
                    dst[c] = (int8_t)(v + (v > 0 ? 0.5f : -0.5f));
                }
            }
        }
    });
}

// GGML quantize_row_q4_0 (the block format cuda_q4_0.go:13-17 uploads).
void mg_quantize_q4_0(const float* w, int rows, int cols, uint8_t* blocks) {
    const size_t nb = (size_t)rows * (cols / 32);
    mg::parallel_for(nb, 1 << 12, [&](size_t b0, size_t b1) {
        for (size_t b = b0; b < b1; b++) {
            const float* x = w + b * 32;
            uint8_t* y = blocks + b * 18;
            float amax = 0.0f, vmax = 0.0f;
            for (int j = 0; j < 32; j++) {
                if (std::fabs(x[j]) > amax) { amax = std::fabs(x[j]); vmax = x[j]; }
            }
            const float d = vmax / -8.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            const uint16_t hd = mg_f32_to_f16(d);
            std::memcpy(y, &hd, 2);
            for (int j = 0; j < 16; j++) {
                int lo = (int8_t)(x[j] * id + 8.5f);
                int hi = (int8_t)(x[j + 16] * id + 8.5f);
                y[2 + j] = (uint8_t)(std::min(lo, 15) | (std::min(hi, 15) << 4));
            }
        }
    });
}

// ---------------------------------------------------------------------------
// Synthetic inputs.  Identical on every machine: integer generator
// (splitmix64 -> xoshiro256**), Marsaglia's polar method, and a logarithm
// written out in plain IEEE double operations (no libm call whose last bit
// could depend on the host CPU).
// ---------------------------------------------------------------------------
namespace {
inline uint64_t splitmix64(uint64_t& s) {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
struct Xoshiro {
    uint64_t s[4];
    Xoshiro(uint64_t seed, uint64_t idx, uint64_t blk) {
        uint64_t k = seed * 0x9e3779b97f4a7c15ull ^ (idx + 0x632be59bd9b4e019ull) * 0xd1342543de82ef95ull ^ (blk << 1 | 1) * 0xa0761d6478bd642full;
        for (int i = 0; i < 4; i++) s[i] = splitmix64(k);
    }
    static inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    inline uint64_t next() {
        const uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]; s[2] ^= t; s[3] = rotl(s[3], 45);
        return r;
    }
    inline double unit() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }   // [0,1)
};
// ln(x) for x in (0, 1]: x = m*2^e, m in [sqrt(.5), sqrt(2)); ln m = 2*atanh((m-1)/(m+1))
inline double det_log(double x) {
    int e;
    double m = std::frexp(x, &e);               // exact
    if (m < 0.70710678118654752440) { m *= 2.0; e -= 1; }
    const double s = (m - 1.0) / (m + 1.0);
    const double z = s * s;
    double p = 1.0 / 23.0;
    p = p * z + 1.0 / 21.0; p = p * z + 1.0 / 19.0; p = p * z + 1.0 / 17.0; p = p * z + 1.0 / 15.0;
    p = p * z + 1.0 / 13.0; p = p * z + 1.0 / 11.0; p = p * z + 1.0 / 9.0;  p = p * z + 1.0 / 7.0;
    p = p * z + 1.0 / 5.0;  p = p * z + 1.0 / 3.0;  p = p * z + 1.0;
    return (double)e * 0.69314718055994530942 + 2.0 * s * p;
}
constexpr size_t kSynthBlock = 4096;
}  // namespace

void mg_synth_normal(uint64_t seed, uint64_t idx, float stdv, float* out, size_t n) {
    const size_t nblk = (n + kSynthBlock - 1) / kSynthBlock;
    mg::parallel_for(nblk, 8, [&](size_t b0, size_t b1) {
        for (size_t b = b0; b < b1; b++) {
            Xoshiro g(seed, idx, b);
            size_t a = b * kSynthBlock, e = std::min(n, a + kSynthBlock);
            size_t i = a;
            while (i < e) {
                double u = 2.0 * g.unit() - 1.0, v = 2.0 * g.unit() - 1.0;
                double s = u * u + v * v;
                if (s >= 1.0 || s == 0.0) continue;
                double f = std::sqrt(-2.0 * det_log(s) / s);
                out[i++] = (float)(u * f * (double)stdv);
                if (i < e) out[i++] = (float)(v * f * (double)stdv);
            }
        }
    });
}

void mg_synth_tokens(uint64_t seed, uint64_t idx, int bound, int* out, size_t n) {
    Xoshiro g(seed, idx, 0x7fffffffull);
    for (size_t i = 0; i < n; i++) out[i] = (int)((g.next() >> 11) % (uint64_t)bound);
}

}  // extern "C"
