// A host program without torch or Python that drives libflashoptim_hip.so through include/flashoptim_hip.h only:
// the shape a C, C++, Go (cgo) or Rust (FFI) caller of the boundary would have.  It allocates with hipMalloc,
// runs three fused AdamW steps on one tensor and on a three-tensor chunked launch, and compares with the scalar C
// restatement of the reference's algorithm (oracle/libfo_oracle.so, loaded with dlopen: test infrastructure).
//
// Checks: narrow parameters within one bf16 ulp; 8-bit codes never more than one step apart and differing on
// fewer than 1 % of the elements (the first steps from a zero state with bf16 gradients sit on rounding
// boundaries unusually often; the Python parity tests apply the exact rounding-tie analysis); fp16 scales at most
// one ulp apart; the multi-tensor launch bit-identical to per-tensor launches; error codes for bad arguments.
// Exit status 0 and a final line "selftest ok" on success.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/flashoptim_hip.h"

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("FAIL %s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)
#define REQUIRE(c, ...) do { if (!(c)) { printf("FAIL line %d: ", __LINE__); printf(__VA_ARGS__); printf("\n"); return 1; } } while (0)

typedef void (*oracle_adam_fn)(void*, uint16_t*, void*, uint16_t*, void*, const void*, void*, int64_t, int, int, int,
                               float, float, float, float, float, int, int);

static uint32_t lcg(uint32_t& s) { s = s * 1664525u + 1013904223u; return s; }
static float uniform(uint32_t& s) { return (float)(lcg(s) >> 8) * (1.0f / 16777216.0f) * 2.0f - 1.0f; }
static uint16_t to_bf16(float f) {  // round to nearest even
    uint32_t u; memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }

struct HostTensor {
    int64_t n;
    std::vector<uint16_t> p, g, ms, vs;
    std::vector<int8_t> ecc, m;
    std::vector<uint8_t> v;
    explicit HostTensor(int64_t n_, uint32_t seed) : n(n_), p(n_), g(n_), ms((n_ + 31) / 32), vs((n_ + 31) / 32), ecc(n_), m(n_), v(n_) {
        uint32_t s = seed;
        for (int64_t i = 0; i < n; ++i) p[i] = to_bf16(0.05f * uniform(s));
    }
    void new_grad(uint32_t seed) { uint32_t s = seed; for (int64_t i = 0; i < n; ++i) g[i] = to_bf16(2e-3f * uniform(s)); }
};

struct DevTensor {
    int64_t n; void *p, *g, *ecc, *m, *ms, *v, *vs;
    int alloc(int64_t n_) {
        n = n_; const int64_t groups = (n + 31) / 32;
        HIP_OK(hipMalloc(&p, n * 2)); HIP_OK(hipMalloc(&g, n * 2)); HIP_OK(hipMalloc(&ecc, n)); HIP_OK(hipMalloc(&m, n));
        HIP_OK(hipMalloc(&v, n)); HIP_OK(hipMalloc(&ms, groups * 2)); HIP_OK(hipMalloc(&vs, groups * 2));
        return 0;
    }
    int upload(const HostTensor& h) {
        const int64_t groups = (n + 31) / 32;
        HIP_OK(hipMemcpy(p, h.p.data(), n * 2, hipMemcpyHostToDevice)); HIP_OK(hipMemcpy(g, h.g.data(), n * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(ecc, h.ecc.data(), n, hipMemcpyHostToDevice)); HIP_OK(hipMemcpy(m, h.m.data(), n, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(v, h.v.data(), n, hipMemcpyHostToDevice)); HIP_OK(hipMemcpy(ms, h.ms.data(), groups * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(vs, h.vs.data(), groups * 2, hipMemcpyHostToDevice));
        return 0;
    }
    int download(HostTensor& h) const {
        const int64_t groups = (n + 31) / 32;
        HIP_OK(hipMemcpy(h.p.data(), p, n * 2, hipMemcpyDeviceToHost)); HIP_OK(hipMemcpy(h.ecc.data(), ecc, n, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(h.m.data(), m, n, hipMemcpyDeviceToHost)); HIP_OK(hipMemcpy(h.v.data(), v, n, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(h.ms.data(), ms, groups * 2, hipMemcpyDeviceToHost)); HIP_OK(hipMemcpy(h.vs.data(), vs, groups * 2, hipMemcpyDeviceToHost));
        return 0;
    }
};

// every output bit equal (what fo_adam_step_exact promises)
static int compare_bits(const HostTensor& got, const HostTensor& want, const char* what) {
    REQUIRE(got.p == want.p, "%s: parameters differ", what);
    REQUIRE(got.ecc == want.ecc, "%s: ECC codes differ", what);
    REQUIRE(got.m == want.m && got.v == want.v, "%s: moment codes differ", what);
    REQUIRE(got.ms == want.ms && got.vs == want.vs, "%s: scales differ", what);
    return 0;
}

// tolerances of the folded update on bf16 parameters: parameters within one ulp, codes within one step on fewer than
// 0.01 % of the elements (none when `first_step`), scales within one fp16 ulp
static int compare(const HostTensor& got, const HostTensor& want, const char* what, bool first_step = false) {
    int64_t code_diffs = 0;
    for (int64_t i = 0; i < got.n; ++i) {
        const float a = from_bf16(got.p[i]), b = from_bf16(want.p[i]);
        const int step = std::abs((int)(int16_t)got.p[i] - (int)(int16_t)want.p[i]);  // same sign: adjacent patterns are one ulp apart
        REQUIRE(got.p[i] == want.p[i] || (a * b >= 0.0f && step <= 1), "%s: parameter %lld off by more than one bf16 ulp (%g vs %g)", what, (long long)i, a, b);
        const int dm = std::abs((int)got.m[i] - (int)want.m[i]), dv = std::abs((int)got.v[i] - (int)want.v[i]);
        REQUIRE(dm <= 1 && dv <= 1, "%s: code %lld differs by more than one step", what, (long long)i);
        code_diffs += (dm != 0) + (dv != 0);
    }
    REQUIRE(code_diffs <= (first_step ? 0 : got.n / 5000 + 1), "%s: %lld of %lld codes differ", what, (long long)code_diffs, (long long)(2 * got.n));
    for (size_t i = 0; i < got.ms.size(); ++i) {
        REQUIRE(std::abs((int)got.ms[i] - (int)want.ms[i]) <= 1 && std::abs((int)got.vs[i] - (int)want.vs[i]) <= 1, "%s: scale %zu differs by more than one fp16 ulp", what, i);
    }
    return 0;
}

int main(int argc, char** argv) {
    const char* oracle_path = argc > 1 ? argv[1] : "oracle/libfo_oracle.so";
    void* handle = dlopen(oracle_path, RTLD_NOW);
    REQUIRE(handle != nullptr, "cannot load %s: %s", oracle_path, dlerror());
    oracle_adam_fn oracle_adam = (oracle_adam_fn)dlsym(handle, "fo_oracle_adam_step");
    REQUIRE(oracle_adam != nullptr, "fo_oracle_adam_step not found");

    REQUIRE(fo_version() >= 100, "fo_version %d", fo_version());
    int count = 0;
    HIP_OK(hipGetDeviceCount(&count));
    REQUIRE(count > 0, "no HIP device");
    REQUIRE(fo_device_compute_units(0) > 0, "fo_device_compute_units: %s", fo_last_error());
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    const float lr = 1e-3f, b1 = 0.9f, b2 = 0.999f, eps = 1e-8f, wd = 1e-5f;
    // ---- one tensor, three steps, against the oracle
    const int64_t n = 100000 + 17;
    HostTensor want(n, 1), got(n, 1);
    DevTensor d;
    if (d.alloc(n)) return 1;
    if (d.upload(want)) return 1;
    for (int step = 1; step <= 3; ++step) {
        want.new_grad(100 + step);
        HIP_OK(hipMemcpy(d.g, want.g.data(), n * 2, hipMemcpyHostToDevice));
        int rc = fo_adam_step(d.m, d.ms, d.v, d.vs, d.p, d.g, d.ecc, n, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, step, stream);
        REQUIRE(rc == 0, "fo_adam_step: %d %s", rc, fo_last_error());
        HIP_OK(hipStreamSynchronize(stream));
        oracle_adam(want.m.data(), want.ms.data(), want.v.data(), want.vs.data(), want.p.data(), want.g.data(), want.ecc.data(), n, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, step);
        if (d.download(got)) return 1;
        char what[64]; snprintf(what, sizeof what, "single tensor, step %d", step);
        if (compare(got, want, what, step == 1)) return 1;
        want = got;  // the next step starts from identical inputs on both sides
        want.g.assign(n, 0);
    }
    printf("single-tensor AdamW steps match the C oracle (n = %lld)\n", (long long)n);

    // ---- the same through fo_adam_step_exact: every bit of every output equals the oracle's, free running
    {
        HostTensor ref(n, 2), out(n, 2);
        DevTensor e;
        if (e.alloc(n)) return 1;
        if (e.upload(ref)) return 1;
        for (int step = 1; step <= 3; ++step) {
            ref.new_grad(200 + step);
            HIP_OK(hipMemcpy(e.g, ref.g.data(), n * 2, hipMemcpyHostToDevice));
            int rc = fo_adam_step_exact(e.m, e.ms, e.v, e.vs, e.p, e.g, e.ecc, n, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, step, stream);
            REQUIRE(rc == 0, "fo_adam_step_exact: %d %s", rc, fo_last_error());
            HIP_OK(hipStreamSynchronize(stream));
            oracle_adam(ref.m.data(), ref.ms.data(), ref.v.data(), ref.vs.data(), ref.p.data(), ref.g.data(), ref.ecc.data(), n, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, step);
            if (e.download(out)) return 1;
            out.g = ref.g;
            char what[64]; snprintf(what, sizeof what, "exact update, step %d", step);
            if (compare_bits(out, ref, what)) return 1;
        }
        printf("fo_adam_step_exact equals the C oracle bit for bit over three free-running steps\n");
    }

    // ---- three tensors: chunked multi-tensor launch == per-tensor launches, bit for bit
    const int64_t lens[3] = {5000, 33, 70001};
    std::vector<HostTensor> host; std::vector<DevTensor> a(3), b(3);
    for (int t = 0; t < 3; ++t) {
        host.emplace_back(lens[t], 10 + t); host[t].new_grad(20 + t);
        if (a[t].alloc(lens[t]) || b[t].alloc(lens[t]) || a[t].upload(host[t]) || b[t].upload(host[t])) return 1;
    }
    const int64_t n_chunks = fo_count_chunks(lens, 3, 0);
    REQUIRE(n_chunks == 2 + 1 + 18, "fo_count_chunks gave %lld", (long long)n_chunks);
    std::vector<fo_chunk> chunks(n_chunks);
    REQUIRE(fo_build_chunks(lens, 3, 0, chunks.data(), n_chunks) == n_chunks, "fo_build_chunks: %s", fo_last_error());
    std::vector<fo_tensor_desc> descs(3);
    for (int t = 0; t < 3; ++t) descs[t] = fo_tensor_desc{a[t].p, a[t].g, a[t].ecc, a[t].m, a[t].ms, a[t].v, a[t].vs, lens[t]};
    void *d_descs, *d_chunks;
    HIP_OK(hipMalloc(&d_descs, sizeof(fo_tensor_desc) * 3)); HIP_OK(hipMalloc(&d_chunks, sizeof(fo_chunk) * n_chunks));
    HIP_OK(hipMemcpy(d_descs, descs.data(), sizeof(fo_tensor_desc) * 3, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_chunks, chunks.data(), sizeof(fo_chunk) * n_chunks, hipMemcpyHostToDevice));
    int rc = fo_multi_adam_step((const fo_tensor_desc*)d_descs, 3, (const fo_chunk*)d_chunks, n_chunks, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, 1, stream);
    REQUIRE(rc == 0, "fo_multi_adam_step: %d %s", rc, fo_last_error());
    for (int t = 0; t < 3; ++t) {
        rc = fo_adam_step(b[t].m, b[t].ms, b[t].v, b[t].vs, b[t].p, b[t].g, b[t].ecc, lens[t], FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, 1, stream);
        REQUIRE(rc == 0, "fo_adam_step: %d %s", rc, fo_last_error());
    }
    HIP_OK(hipStreamSynchronize(stream));
    for (int t = 0; t < 3; ++t) {
        HostTensor x(lens[t], 0), y(lens[t], 0);
        if (a[t].download(x) || b[t].download(y)) return 1;
        REQUIRE(x.p == y.p && x.ecc == y.ecc && x.m == y.m && x.v == y.v && x.ms == y.ms && x.vs == y.vs, "multi-tensor launch differs from per-tensor launch on tensor %d", t);
    }
    printf("multi-tensor launch is bit-identical to per-tensor launches\n");

    // ---- error conventions: negative fo_error codes, message available, nothing thrown
    rc = fo_adam_step(d.m, d.ms, d.v, d.vs, d.p, d.g, d.ecc, n, 7, 1, 1, lr, b1, b2, eps, wd, 1, 1, stream);
    REQUIRE(rc < 0 && strlen(fo_last_error()) > 0, "bad dtype accepted (rc %d)", rc);
    rc = fo_adam_step(d.m, nullptr, d.v, d.vs, d.p, d.g, d.ecc, n, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, 1, stream);
    REQUIRE(rc < 0, "NULL scales accepted (rc %d)", rc);
    rc = fo_adam_step(d.m, d.ms, d.v, d.vs, d.p, d.g, d.ecc, 0, FO_BF16, 1, 1, lr, b1, b2, eps, wd, 1, 1, stream);
    REQUIRE(rc == 0, "n == 0 must be a no-op (rc %d)", rc);
    printf("selftest ok\n");
    return 0;
}
