// C++ host-side check of libssd_hip through include/ssd_hip.hpp: the calls a compiled host program makes
// (forward, streaming continuation step by step and as one call, error paths), each checked against the plain-C oracle
// (oracle/ssd_oracle.c, linked from oracle/libssd_oracle.so).  Run by tests/test_gpu_host_cpp.py on the GPU.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "ssd_hip.hpp"

extern "C" int ssd_oracle_seq_f64(int64_t Bsz, int64_t L, int64_t H, int64_t P, int64_t N, int64_t G, const double *x,
                                  const double *dt, const double *A, const double *Bm, const double *Cm, const double *D,
                                  const double *init, double *y, double *final_state, int nthreads);

namespace {

struct Rng {  // xorshift64* and Box-Muller: fixed inputs without any library's generator
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 1) {}
    double uniform() {
        s ^= s >> 12; s ^= s << 25; s ^= s >> 27;
        return (double)((s * 0x2545F4914F6CDD1Dull) >> 11) / 9007199254740992.0;
    }
    double normal() {
        const double u1 = uniform() + 1e-300, u2 = uniform();
        return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
    }
};

uint16_t to_bf16(float f) {  // round to nearest even
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float from_bf16(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

struct Problem {
    int64_t B, L, H, P, N, G, chunk;
    bool bf16;
    std::vector<double> x, dt, A, Bm, Cm, D;  // the exact values the device sees
};

Problem make(int64_t B, int64_t L, int64_t H, int64_t P, int64_t N, int64_t G, int64_t chunk, bool bf16, uint64_t seed) {
    Problem p{B, L, H, P, N, G, chunk, bf16, {}, {}, {}, {}, {}, {}};
    Rng r(seed);
    auto q = [&](double v) { return bf16 ? (double)from_bf16(to_bf16((float)v)) : (double)(float)v; };
    p.x.resize(B * L * H * P);
    for (auto &v : p.x) v = q(r.normal());
    p.dt.resize(B * L * H);
    for (auto &v : p.dt) v = q(std::log1p(std::exp(r.normal() - 2.0)));
    p.A.resize(H);
    for (auto &v : p.A) v = (double)(float)(-std::exp(r.uniform() * std::log(16.0)));
    p.Bm.resize(B * L * G * N);
    for (auto &v : p.Bm) v = q(r.normal() / std::sqrt((double)N));
    p.Cm.resize(B * L * G * N);
    for (auto &v : p.Cm) v = q(r.normal() / std::sqrt((double)N));
    p.D.resize(H);
    for (auto &v : p.D) v = (double)(float)r.normal();
    return p;
}

ssd_hip::DeviceBuffer upload(const std::vector<double> &v, bool bf16) {
    if (bf16) {
        std::vector<uint16_t> h(v.size());
        for (size_t i = 0; i < v.size(); ++i) h[i] = to_bf16((float)v[i]);
        ssd_hip::DeviceBuffer d(h.size() * 2);
        d.upload(h.data(), h.size() * 2);
        return d;
    }
    std::vector<float> h(v.begin(), v.end());
    ssd_hip::DeviceBuffer d(h.size() * 4);
    d.upload(h.data(), h.size() * 4);
    return d;
}

std::vector<double> download(const ssd_hip::DeviceBuffer &d, size_t n, bool bf16) {
    std::vector<double> out(n);
    if (bf16) {
        std::vector<uint16_t> h(n);
        d.download(h.data(), n * 2);
        for (size_t i = 0; i < n; ++i) out[i] = from_bf16(h[i]);
    } else {
        std::vector<float> h(n);
        d.download(h.data(), n * 4);
        for (size_t i = 0; i < n; ++i) out[i] = h[i];
    }
    return out;
}

// max over elements of |out - ref| / (tol * rms(ref) + one rounding of ref in the output format)
double worst(const std::vector<double> &out, const std::vector<double> &ref, double tol, bool bf16_out) {
    double ss = 0;
    for (double v : ref) ss += v * v;
    const double rms = std::sqrt(ss / (double)ref.size());
    double w = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        const double allowed = tol * rms + (bf16_out ? std::ldexp(std::fabs(ref[i]), -8) : 0.0);
        w = std::fmax(w, std::fabs(out[i] - ref[i]) / allowed);
    }
    return w;
}

int failures = 0;
void expect(bool ok, const char *what) {
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    if (!ok) ++failures;
}

void forward_case(const Problem &p, const char *name) {
    using namespace ssd_hip;
    const DType t = p.bf16 ? DType::BF16 : DType::F32;
    DeviceBuffer x = upload(p.x, p.bf16), dt = upload(p.dt, p.bf16), A = upload(p.A, false), Bm = upload(p.Bm, p.bf16),
                 Cm = upload(p.Cm, p.bf16), D = upload(p.D, false);
    const TensorView vx = view(x.data(), t, {p.B, p.L, p.H, p.P}), vdt = view(dt.data(), t, {p.B, p.L, p.H}),
                     vA = view(A.data(), DType::F32, {p.H}), vB = view(Bm.data(), t, {p.B, p.L, p.G, p.N}),
                     vC = view(Cm.data(), t, {p.B, p.L, p.G, p.N}), vD = view(D.data(), DType::F32, {p.H});
    std::vector<double> y(p.x.size()), fin(p.B * p.H * p.P * p.N);
    ssd_oracle_seq_f64(p.B, p.L, p.H, p.P, p.N, p.G, p.x.data(), p.dt.data(), p.A.data(), p.Bm.data(), p.Cm.data(), p.D.data(),
                       nullptr, y.data(), fin.data(), 8);
    const double tol = p.bf16 ? 2e-2 : 1e-4;
    ScanOutput out = ssd_chunk_scan(vx, vdt, vA, vB, vC, &vD, p.chunk, nullptr);
    char what[160];
    const double wy = worst(download(out.y, y.size(), p.bf16), y, tol, p.bf16);
    const double wf = worst(download(out.final_states, fin.size(), false), fin, tol, false);
    std::snprintf(what, sizeof(what), "%s: forward y %.3f and final state %.3f of the allowance", name, wy, wf);
    expect(wy <= 1.0 && wf <= 1.0, what);

    // streaming continuation: scan a prefix, adopt its final state, step through the rest
    const int64_t tail = 8, pre = p.L - tail;
    std::vector<double> px(p.B * pre * p.H * p.P), pdt(p.B * pre * p.H), pB(p.B * pre * p.G * p.N), pC(pB.size());
    for (int64_t b = 0; b < p.B; ++b) {
        std::copy_n(&p.x[b * p.L * p.H * p.P], pre * p.H * p.P, &px[b * pre * p.H * p.P]);
        std::copy_n(&p.dt[b * p.L * p.H], pre * p.H, &pdt[b * pre * p.H]);
        std::copy_n(&p.Bm[b * p.L * p.G * p.N], pre * p.G * p.N, &pB[b * pre * p.G * p.N]);
        std::copy_n(&p.Cm[b * p.L * p.G * p.N], pre * p.G * p.N, &pC[b * pre * p.G * p.N]);
    }
    DeviceBuffer dpx = upload(px, p.bf16), dpdt = upload(pdt, p.bf16), dpB = upload(pB, p.bf16), dpC = upload(pC, p.bf16);
    ScanOutput prefix = ssd_chunk_scan(view(dpx.data(), t, {p.B, pre, p.H, p.P}), view(dpdt.data(), t, {p.B, pre, p.H}), vA,
                                       view(dpB.data(), t, {p.B, pre, p.G, p.N}), view(dpC.data(), t, {p.B, pre, p.G, p.N}), &vD,
                                       p.chunk, nullptr);
    StreamState state(p.B, p.H, p.P, p.N);
    state.adopt(prefix.final_states);
    double ws = 0;
    for (int64_t s = 0; s < tail; ++s) {
        const int64_t tt = pre + s;
        std::vector<double> sx(p.B * p.H * p.P), sdt(p.B * p.H), sB(p.B * p.G * p.N), sC(sB.size()), sy(sx.size());
        for (int64_t b = 0; b < p.B; ++b) {
            std::copy_n(&p.x[(b * p.L + tt) * p.H * p.P], p.H * p.P, &sx[b * p.H * p.P]);
            std::copy_n(&p.dt[(b * p.L + tt) * p.H], p.H, &sdt[b * p.H]);
            std::copy_n(&p.Bm[(b * p.L + tt) * p.G * p.N], p.G * p.N, &sB[b * p.G * p.N]);
            std::copy_n(&p.Cm[(b * p.L + tt) * p.G * p.N], p.G * p.N, &sC[b * p.G * p.N]);
            std::copy_n(&y[(b * p.L + tt) * p.H * p.P], p.H * p.P, &sy[b * p.H * p.P]);
        }
        DeviceBuffer dx = upload(sx, p.bf16), ddt = upload(sdt, p.bf16), dB = upload(sB, p.bf16), dC = upload(sC, p.bf16);
        DeviceBuffer ys = ssd_step(state, view(dx.data(), t, {p.B, p.H, p.P}), view(ddt.data(), t, {p.B, p.H}), vA,
                                   view(dB.data(), t, {p.B, p.G, p.N}), view(dC.data(), t, {p.B, p.G, p.N}), &vD);
        check_hip(hipDeviceSynchronize(), "sync");
        ws = std::fmax(ws, worst(download(ys, sy.size(), p.bf16), sy, tol, p.bf16));
    }
    std::vector<float> st(fin.size());
    check_hip(hipMemcpy(st.data(), state.data(), st.size() * 4, hipMemcpyDeviceToHost), "state");
    const double wst = worst(std::vector<double>(st.begin(), st.end()), fin, tol, false);
    std::snprintf(what, sizeof(what), "%s: prefix + %d steps == full scan: y %.3f, state %.3f of the allowance", name, (int)tail, ws, wst);
    expect(ws <= 1.0 && wst <= 1.0, what);

    // the same continuation as one call over a longer tail (bf16 runs of 16 steps or more go to the scan kernel)
    {
        const int64_t tail2 = 24, pre2 = p.L - tail2;
        std::vector<double> qx(p.B * pre2 * p.H * p.P), qdt(p.B * pre2 * p.H), qB(p.B * pre2 * p.G * p.N), qC(qB.size());
        std::vector<double> tx(p.B * tail2 * p.H * p.P), tdt(p.B * tail2 * p.H), tB(p.B * tail2 * p.G * p.N), tC(tB.size()),
            ty(tx.size());
        for (int64_t b = 0; b < p.B; ++b) {
            std::copy_n(&p.x[b * p.L * p.H * p.P], pre2 * p.H * p.P, &qx[b * pre2 * p.H * p.P]);
            std::copy_n(&p.dt[b * p.L * p.H], pre2 * p.H, &qdt[b * pre2 * p.H]);
            std::copy_n(&p.Bm[b * p.L * p.G * p.N], pre2 * p.G * p.N, &qB[b * pre2 * p.G * p.N]);
            std::copy_n(&p.Cm[b * p.L * p.G * p.N], pre2 * p.G * p.N, &qC[b * pre2 * p.G * p.N]);
            std::copy_n(&p.x[(b * p.L + pre2) * p.H * p.P], tail2 * p.H * p.P, &tx[b * tail2 * p.H * p.P]);
            std::copy_n(&p.dt[(b * p.L + pre2) * p.H], tail2 * p.H, &tdt[b * tail2 * p.H]);
            std::copy_n(&p.Bm[(b * p.L + pre2) * p.G * p.N], tail2 * p.G * p.N, &tB[b * tail2 * p.G * p.N]);
            std::copy_n(&p.Cm[(b * p.L + pre2) * p.G * p.N], tail2 * p.G * p.N, &tC[b * tail2 * p.G * p.N]);
            std::copy_n(&y[(b * p.L + pre2) * p.H * p.P], tail2 * p.H * p.P, &ty[b * tail2 * p.H * p.P]);
        }
        DeviceBuffer dqx = upload(qx, p.bf16), dqdt = upload(qdt, p.bf16), dqB = upload(qB, p.bf16), dqC = upload(qC, p.bf16);
        ScanOutput head = ssd_chunk_scan(view(dqx.data(), t, {p.B, pre2, p.H, p.P}), view(dqdt.data(), t, {p.B, pre2, p.H}), vA,
                                         view(dqB.data(), t, {p.B, pre2, p.G, p.N}), view(dqC.data(), t, {p.B, pre2, p.G, p.N}),
                                         &vD, p.chunk, nullptr);
        StreamState many(p.B, p.H, p.P, p.N);
        many.adopt(head.final_states);
        DeviceBuffer dtx = upload(tx, p.bf16), dtdt = upload(tdt, p.bf16), dtB = upload(tB, p.bf16), dtC = upload(tC, p.bf16);
        DeviceBuffer ym = ssd_steps(many, view(dtx.data(), t, {p.B, tail2, p.H, p.P}), view(dtdt.data(), t, {p.B, tail2, p.H}), vA,
                                    view(dtB.data(), t, {p.B, tail2, p.G, p.N}), view(dtC.data(), t, {p.B, tail2, p.G, p.N}), &vD);
        check_hip(hipDeviceSynchronize(), "sync");
        const double wm = worst(download(ym, ty.size(), p.bf16), ty, tol, p.bf16);
        std::vector<float> sm(fin.size());
        check_hip(hipMemcpy(sm.data(), many.data(), sm.size() * 4, hipMemcpyDeviceToHost), "state");
        const double wms = worst(std::vector<double>(sm.begin(), sm.end()), fin, tol, false);
        std::snprintf(what, sizeof(what), "%s: prefix + %d steps in one call == full scan: y %.3f, state %.3f of the allowance",
                      name, (int)tail2, wm, wms);
        expect(wm <= 1.0 && wms <= 1.0, what);
    }

    // a reset stream row starts from the empty state again
    state.reset_row(1);
    std::vector<float> row(p.H * p.P * p.N);
    check_hip(hipMemcpy(row.data(), state.data() + row.size(), row.size() * 4, hipMemcpyDeviceToHost), "row");
    bool zero = true;
    for (float v : row) zero = zero && v == 0.f;
    expect(zero, "reset_row zeroes one stream and only that one");
}

void error_cases() {
    using namespace ssd_hip;
    const Problem p = make(2, 64, 4, 16, 16, 1, 64, false, 5);
    DeviceBuffer x = upload(p.x, false), dt = upload(p.dt, false), A = upload(p.A, false), Bm = upload(p.Bm, false),
                 Cm = upload(p.Cm, false);
    const TensorView vx = view(x.data(), DType::F32, {p.B, p.L, p.H, p.P}), vdt = view(dt.data(), DType::F32, {p.B, p.L, p.H}),
                     vA = view(A.data(), DType::F32, {p.H}), vB = view(Bm.data(), DType::F32, {p.B, p.L, p.G, p.N}),
                     vC = view(Cm.data(), DType::F32, {p.B, p.L, p.G, p.N});
    try {
        ssd_chunk_scan(vx, view(dt.data(), DType::F32, {p.B, p.L, p.H + 1}), vA, vB, vC, nullptr, 64, nullptr);
        expect(false, "a dt of the wrong shape is refused");
    } catch (const Error &e) {
        expect(e.code() == SSD_ERR_INVALID && std::strstr(e.what(), "dt") != nullptr, "a dt of the wrong shape is refused by the wrapper");
    }
    try {
        ssd_chunk_scan(vx, vdt, vA, vB, vC, nullptr, 48, nullptr);
        expect(false, "an unsupported chunk is refused");
    } catch (const Error &e) {
        expect(e.code() == SSD_ERR_UNSUPPORTED && std::strstr(e.what(), "chunk") != nullptr,
               "an unsupported chunk is refused by the library, with its message");
    }
    char *leftover = ssd_get_and_reset_last_err();
    expect(leftover == nullptr, "the error slot is empty after the message was taken");
    std::free(leftover);
}

}  // namespace

int main() {
    try {
        std::printf("libssd_hip version %d\n", ssd_version());
        forward_case(make(4, 256, 4, 16, 16, 1, 64, false, 0), "plumbing shape, float32");
        forward_case(make(8, 300, 8, 32, 64, 1, 128, true, 1), "policy heads, bf16, ragged length");
        forward_case(make(3, 200, 4, 64, 32, 2, 64, false, 2), "groups, float32");
        error_cases();
    } catch (const std::exception &e) {
        std::printf("FAIL unexpected exception: %s\n", e.what());
        return 2;
    }
    std::printf(failures == 0 ? "host_check OK\n" : "host_check FAILED (%d)\n", failures);
    return failures == 0 ? 0 : 1;
}
