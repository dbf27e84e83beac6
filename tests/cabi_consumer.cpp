// A consumer of liblpmm_hip.so that knows nothing of Python or torch: it includes only
// include/lpmm_hip.h and the HIP runtime API, owns its device memory, and checks what the
// library leaves there against the CPU oracle (oracle/lpmm_oracle.c, linked in as the
// checker).  It is what a binding of another host language would do through its FFI:
// plain pointers, sizes, a stream, integer status codes.
//
// Covered: the fused 4-bit step (single tensor, ragged last group; multi-tensor table with
// per-tensor step counts), the fp32-state step, group-128 quantise -> dequantise, and the
// error codes for bad arguments, which must come back without any launch.
//
// Build: make -C tests (g++ for this file, gcc for the oracle, linked against liblpmm_hip.so
// and libamdhip64.so; __graft_entry__.build() runs it).
// Exit status 0 and a final line "cabi consumer ok" mean every check passed.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "lpmm_hip.h"

extern "C" {
// the checker's entry points (oracle/lpmm_oracle.c)
void lpmm_oracle_adamw4bit_step(float *p, const float *g, uint8_t *m_codes, uint8_t *v_codes, float *m_scale,
                                float *v_scale, const float *qmap_m, const float *qmap_v, int64_t n, float beta1,
                                float beta2, float lr, float weight_decay, float eps, float step);
void lpmm_oracle_adamw_fp32_step(float *p, const float *g, float *m, float *v, int64_t n, float beta1, float beta2,
                                 float lr, float weight_decay, float eps, float step);
void lpmm_oracle_quant_group(const float *x, int64_t n, int64_t gp_sz, const float *qmap, uint8_t *codes,
                             float *max1);
void lpmm_oracle_dequant_group(const uint8_t *codes, const float *max1, const float *qmap, int64_t n, int64_t gp_sz,
                               float *out);
}

namespace {

// the reference's two 4-bit maps (lpmm/functional.py:244-268 with the shipped configuration:
// signed dynamic-exponent map for m, linear map without zero for v), as bit patterns
const uint32_t kQmapMBits[16] = {0xbf633333u, 0xbf29999au, 0xbee00000u, 0xbe599999u, 0xbd9eb852u, 0xbd051eb9u,
                                 0xbbb43958u, 0x00000000u, 0x3bb43958u, 0x3d051eb9u, 0x3d9eb852u, 0x3e599999u,
                                 0x3ee00000u, 0x3f29999au, 0x3f633333u, 0x3f800000u};

int failures = 0;

#define CHECK(cond, ...)                               \
    do {                                               \
        if (!(cond)) {                                 \
            ++failures;                                \
            std::printf("FAILED %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                  \
            std::printf("\n");                         \
        }                                              \
    } while (0)

#define HIP_OK(call)                                                                  \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                       \
            std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                             \
        }                                                                             \
    } while (0)

// deterministic inputs: a 64-bit LCG, two uniforms -> one normal (Box-Muller)
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 1) {}
    double uniform()
    {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        return ((s >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    }
    float normal() { return (float)(std::sqrt(-2.0 * std::log(uniform())) * std::cos(6.283185307179586 * uniform())); }
};

template <class T>
struct DeviceBuf {
    T *d = nullptr;
    size_t count = 0;
    explicit DeviceBuf(size_t n) : count(n) { HIP_OK(hipMalloc(reinterpret_cast<void **>(&d), n * sizeof(T) + 16)); }
    DeviceBuf(const DeviceBuf &) = delete;
    DeviceBuf &operator=(const DeviceBuf &) = delete;
    ~DeviceBuf() { (void)hipFree(d); }
    void upload(const std::vector<T> &h) { HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
    std::vector<T> download() const
    {
        std::vector<T> h(count);
        HIP_OK(hipMemcpy(h.data(), d, count * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

// host and device copy of one tensor's fused-path state
struct Tensor4 {
    int64_t n;
    std::vector<float> p, g, ms, vs;
    std::vector<float> p_before;  // the parameters the last step started from
    std::vector<uint8_t> mc, vc;
    DeviceBuf<float> dp, dg, dms, dvs;
    DeviceBuf<uint8_t> dmc, dvc;
    explicit Tensor4(int64_t n_)
        : n(n_), p(n_), g(n_), ms((n_ + 127) / 128, 0.0f), vs((n_ + 127) / 128, 0.0f), mc((n_ + 1) / 2, 0),
          vc((n_ + 1) / 2, 0), dp(n_), dg(n_), dms(ms.size()), dvs(vs.size()), dmc(mc.size()), dvc(vc.size())
    {
    }
    void upload_all()
    {
        dp.upload(p); dg.upload(g); dms.upload(ms); dvs.upload(vs); dmc.upload(mc); dvc.upload(vc);
    }
};

// Codes and scales bit for bit; parameters within 1e-6 of the larger of the parameter before and after
// the step (the library computes the update term with the hardware's sqrt and reciprocal).  The device
// parameters are then replaced by the oracle's, so that the next step starts from identical inputs.
void compare_tensor(Tensor4 &t, const char *what)
{
    const std::vector<float> p = t.dp.download(), ms = t.dms.download(), vs = t.dvs.download();
    const std::vector<uint8_t> mc = t.dmc.download(), vc = t.dvc.download();
    CHECK(std::memcmp(mc.data(), t.mc.data(), mc.size()) == 0, "%s: m codes differ from the oracle", what);
    CHECK(std::memcmp(vc.data(), t.vc.data(), vc.size()) == 0, "%s: v codes differ from the oracle", what);
    CHECK(std::memcmp(ms.data(), t.ms.data(), ms.size() * 4) == 0, "%s: m scales differ from the oracle", what);
    CHECK(std::memcmp(vs.data(), t.vs.data(), vs.size() * 4) == 0, "%s: v scales differ from the oracle", what);
    double worst = 0.0;
    for (int64_t i = 0; i < t.n; ++i) {
        const double yard = std::fmax(std::fmax(std::fabs((double)t.p[i]), std::fabs((double)t.p_before[i])), 1e-30);
        worst = std::fmax(worst, std::fabs((double)p[i] - (double)t.p[i]) / yard);
    }
    CHECK(worst <= 1e-6, "%s: parameters differ from the oracle by %.3e relative (tolerance 1e-6)", what, worst);
    t.dp.upload(t.p);
}

const float kBeta1 = 0.9f, kBeta2 = 0.999f, kLr = 1e-3f, kWd = 0.01f, kEps = 1e-8f;

}  // namespace

int main()
{
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices < 1) {
        std::printf("no GPU\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));
    CHECK(lpmm_abi_version() == LPMM_HIP_ABI_VERSION, "ABI version %d, header %d", lpmm_abi_version(),
          LPMM_HIP_ABI_VERSION);

    float qm[16], qv[16];
    std::memcpy(qm, kQmapMBits, sizeof(qm));
    for (int k = 0; k < 16; ++k)
        qv[k] = (float)(k + 1) / 16.0f;  // 1/16, 2/16, ..., 16/16: every entry exact
    DeviceBuf<float> dqm(16), dqv(16);
    dqm.upload(std::vector<float>(qm, qm + 16));
    dqv.upload(std::vector<float>(qv, qv + 16));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    // ---- bad arguments come back as status codes, before any launch -----------------------
    {
        DeviceBuf<float> x(256);
        DeviceBuf<uint8_t> c(256);
        CHECK(lpmm_adamw4bit_step(nullptr, x.d, c.d, c.d, x.d, x.d, dqm.d, dqv.d, 256, kBeta1, kBeta2, kLr, kWd, kEps,
                                  1.0f, stream) == LPMM_ERR_NULL, "NULL p not reported");
        CHECK(lpmm_adamw4bit_step(x.d, x.d, c.d, c.d, x.d, x.d, dqm.d, dqv.d, -1, kBeta1, kBeta2, kLr, kWd, kEps,
                                  1.0f, stream) == LPMM_ERR_SIZE, "negative n not reported");
        CHECK(lpmm_adamw4bit_step(reinterpret_cast<float *>(reinterpret_cast<char *>(x.d) + 1), x.d, c.d, c.d, x.d,
                                  x.d, dqm.d, dqv.d, 128, kBeta1, kBeta2, kLr, kWd, kEps, 1.0f, stream) ==
                  LPMM_ERR_ALIGN, "misaligned p not reported");
        CHECK(std::strlen(lpmm_status_string(LPMM_ERR_ALIGN)) > 0, "no text for a status");
        CHECK(hipGetLastError() == hipSuccess, "a rejected call touched the HIP runtime");
    }

    // ---- fused step, one tensor at a time: whole tiles, a ragged last group, a tiny tensor --
    const int64_t sizes[] = {8320, 4 * 2048 * 37 + 66, 4098, 131072 * 3};
    std::vector<Tensor4 *> tensors;
    Rng rng(2024);
    for (int64_t n : sizes) {
        Tensor4 *t = new Tensor4(n);
        for (int64_t i = 0; i < n; ++i)
            t->p[i] = rng.normal() * 0.02f;
        tensors.push_back(t);
    }
    for (int step = 1; step <= 3; ++step) {
        for (Tensor4 *t : tensors) {
            for (int64_t i = 0; i < t->n; ++i)
                t->g[i] = rng.normal() * 1e-3f * (1.0f + 20.0f * (float)(i % 977 == 0));
            if (step == 1)
                t->upload_all();
            else
                t->dg.upload(t->g);
            const int st = lpmm_adamw4bit_step(t->dp.d, t->dg.d, t->dmc.d, t->dvc.d, t->dms.d, t->dvs.d, dqm.d, dqv.d,
                                               t->n, kBeta1, kBeta2, kLr, kWd, kEps, (float)step, stream);
            CHECK(st == LPMM_OK, "lpmm_adamw4bit_step: %s", lpmm_status_string(st));
            t->p_before = t->p;
            lpmm_oracle_adamw4bit_step(t->p.data(), t->g.data(), t->mc.data(), t->vc.data(), t->ms.data(),
                                       t->vs.data(), qm, qv, t->n, kBeta1, kBeta2, kLr, kWd, kEps, (float)step);
        }
        HIP_OK(hipStreamSynchronize(stream));
        for (Tensor4 *t : tensors) {
            char what[96];
            std::snprintf(what, sizeof(what), "single-tensor step %d, n = %lld", step, (long long)t->n);
            compare_tensor(*t, what);
        }
    }

    // ---- the same tensors through the multi-tensor table, each with its own step count -------
    {
        std::vector<lpmm_adamw4bit_tensor> table;
        int k = 0;
        for (Tensor4 *t : tensors) {
            for (int64_t i = 0; i < t->n; ++i)
                t->g[i] = rng.normal() * 1e-3f;
            t->dg.upload(t->g);
            const float step = 4.0f + (float)k++;
            lpmm_adamw4bit_tensor rec = {t->dp.d, t->dg.d, t->dmc.d, t->dvc.d, t->dms.d, t->dvs.d, t->n, step, 0.0f};
            table.push_back(rec);
            t->p_before = t->p;
            lpmm_oracle_adamw4bit_step(t->p.data(), t->g.data(), t->mc.data(), t->vc.data(), t->ms.data(),
                                       t->vs.data(), qm, qv, t->n, kBeta1, kBeta2, kLr, kWd, kEps, step);
        }
        const int st = lpmm_adamw4bit_step_multi(table.data(), (int64_t)table.size(), dqm.d, dqv.d, kBeta1, kBeta2,
                                                 kLr, kWd, kEps, stream);
        CHECK(st == LPMM_OK, "lpmm_adamw4bit_step_multi: %s", lpmm_status_string(st));
        HIP_OK(hipStreamSynchronize(stream));
        for (Tensor4 *t : tensors)
            compare_tensor(*t, "multi-tensor step");
        CHECK(lpmm_adamw4bit_step_multi(table.data(), 0, dqm.d, dqv.d, kBeta1, kBeta2, kLr, kWd, kEps, stream) ==
                  LPMM_OK, "an empty table is not an error");
    }
    for (Tensor4 *t : tensors)
        delete t;

    // ---- fp32-state step (tensors at or under the quantisation threshold) ---------------------
    {
        const int64_t n = 4096;
        std::vector<float> p(n), g(n), m(n, 0.0f), v(n, 0.0f);
        for (int64_t i = 0; i < n; ++i) {
            p[i] = rng.normal() * 0.02f;
            g[i] = rng.normal() * 1e-3f;
        }
        DeviceBuf<float> dp(n), dg(n), dm(n), dv(n);
        dp.upload(p); dg.upload(g); dm.upload(m); dv.upload(v);
        for (int step = 1; step <= 2; ++step) {
            const int st = lpmm_adamw_fp32_step(dp.d, dg.d, dm.d, dv.d, n, kBeta1, kBeta2, kLr, kWd, kEps, (float)step,
                                                stream);
            CHECK(st == LPMM_OK, "lpmm_adamw_fp32_step: %s", lpmm_status_string(st));
            lpmm_oracle_adamw_fp32_step(p.data(), g.data(), m.data(), v.data(), n, kBeta1, kBeta2, kLr, kWd, kEps,
                                        (float)step);
        }
        HIP_OK(hipStreamSynchronize(stream));
        const std::vector<float> gm = dm.download(), gv = dv.download(), gp = dp.download();
        CHECK(std::memcmp(gm.data(), m.data(), n * 4) == 0, "fp32-state step: m differs from the oracle");
        CHECK(std::memcmp(gv.data(), v.data(), n * 4) == 0, "fp32-state step: v differs from the oracle");
        double worst = 0.0;
        for (int64_t i = 0; i < n; ++i)
            worst = std::fmax(worst, std::fabs((double)gp[i] - (double)p[i]) / std::fmax(std::fabs((double)p[i]), 1e-30));
        CHECK(worst <= 1e-6, "fp32-state step: parameters differ by %.3e relative", worst);
    }

    // ---- group-128 quantise -> dequantise in the non-fused packed layout ----------------------
    {
        const int64_t n = 2048 * 9 + 300, gp = 128, groups = (n + gp - 1) / gp;
        const int64_t nbytes = (groups * gp + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * (LPMM_PACK_GROUP / 2) + 1;
        std::vector<float> x(n), max1(groups), back(n);
        std::vector<uint8_t> codes(nbytes);
        for (int64_t i = 0; i < n; ++i)
            x[i] = rng.normal() * (i % 513 == 0 ? 30.0f : 1.0f);
        DeviceBuf<float> dx(n), dmax(groups), dback(n);
        DeviceBuf<uint8_t> dcodes(nbytes);
        dx.upload(x);
        int st = lpmm_quant_group(dx.d, n, gp, dqm.d, dcodes.d, dmax.d, stream);
        CHECK(st == LPMM_OK, "lpmm_quant_group: %s", lpmm_status_string(st));
        st = lpmm_dequant_group(dcodes.d, dmax.d, dqm.d, n, gp, dback.d, stream);
        CHECK(st == LPMM_OK, "lpmm_dequant_group: %s", lpmm_status_string(st));
        HIP_OK(hipStreamSynchronize(stream));
        lpmm_oracle_quant_group(x.data(), n, gp, qm, codes.data(), max1.data());
        lpmm_oracle_dequant_group(codes.data(), max1.data(), qm, n, gp, back.data());
        const std::vector<uint8_t> gc = dcodes.download();
        const std::vector<float> gmx = dmax.download(), gb = dback.download();
        CHECK(std::memcmp(gc.data(), codes.data(), nbytes) == 0, "group quantise: codes differ from the oracle");
        CHECK(std::memcmp(gmx.data(), max1.data(), groups * 4) == 0, "group quantise: scales differ from the oracle");
        CHECK(std::memcmp(gb.data(), back.data(), n * 4) == 0, "group dequantise: values differ from the oracle");
    }

    HIP_OK(hipStreamDestroy(stream));
    if (failures) {
        std::printf("%d check(s) failed\n", failures);
        return 1;
    }
    std::printf("cabi consumer ok\n");
    return 0;
}
