// TEST INFRASTRUCTURE.  A program without Python or PyTorch that drives the C ABI of include/ps_adam.h the way a
// host application written in C or C++ would: device memory from hipMalloc, a stream from hipStreamCreate, chunk
// descriptors as a plain host array, pinned host memory from hipHostMalloc for host-resident chunks.  Every result is compared bit for bit with the CPU restatement of the
// reference operator (oracle/adam_oracle.c, linked as liboracle_adam.so) and, for the loss-scale decisions, with
// the rules of patrickstar/fp16/loss_scaler.py:158-182 written out below.
//
// Built by tests/c_abi/Makefile on the CPU (host code only); run by tests/test_c_abi_gpu.py on a GPU.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ps_adam.h"

extern "C" {
// oracle/adam_oracle.c
struct oracle_adam_opaque {
    unsigned char bytes[128];
};
int oracle_sizeof_state(void);
void oracle_adam_init(void* o, float lr, float beta1, float beta2, float eps, float weight_decay, int adamw);
void oracle_adam_advance(void* o, uint64_t step, float beta1, float beta2);
void oracle_adam_set(void* o, float lr, float eps, float weight_decay, int bias_correction);
int oracle_adam_span(const void* o, float* p, const void* g, int g_half, float* m, float* v, size_t n,
                     float loss_scale, int isa);
void oracle_cast_f32_to_f16(const float* src, uint16_t* dst, size_t n);
uint16_t oracle_f32_to_f16(float f);
}

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s failed: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__); \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)
#define PS_OK(call)                                                                        \
    do {                                                                                   \
        int rc_ = (call);                                                                  \
        if (rc_ != 0) {                                                                    \
            fprintf(stderr, "%s returned %d: %s (line %d)\n", #call, rc_, ps_last_error(), __LINE__); \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)

namespace {

struct Lcg {  // deterministic inputs without any library
    uint64_t s;
    double uniform() { s = s * 6364136223846793005ull + 1442695040888963407ull; return ((s >> 11) + 0.5) / 9007199254740992.0; }
    double normal() { return std::sqrt(-2.0 * std::log(uniform())) * std::cos(6.283185307179586 * uniform()); }
};

struct HostChunk {
    std::vector<float> p, m, v;
    std::vector<uint16_t> h;
};

struct DeviceChunk {
    float *p = nullptr, *m = nullptr, *v = nullptr;
    uint16_t* h = nullptr;
};

int upload(const HostChunk& c, DeviceChunk& d, size_t n)
{
    HIP_OK(hipMemcpy(d.p, c.p.data(), n * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.m, c.m.data(), n * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.v, c.v.data(), n * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.h, c.h.data(), n * 2, hipMemcpyHostToDevice));
    return 0;
}

int compare(const HostChunk& want, const DeviceChunk& d, size_t n, const char* what, int chunk)
{
    std::vector<float> f(n);
    std::vector<uint16_t> h(n);
    const float* src[3] = {d.p, d.m, d.v};
    const std::vector<float>* ref[3] = {&want.p, &want.m, &want.v};
    const char* name[3] = {"fp32 param", "exp_avg", "exp_avg_sq"};
    for (int k = 0; k < 3; ++k) {
        HIP_OK(hipMemcpy(f.data(), src[k], n * 4, hipMemcpyDeviceToHost));
        if (memcmp(f.data(), ref[k]->data(), n * 4) != 0) {
            fprintf(stderr, "%s: chunk %d %s differs from the CPU restatement\n", what, chunk, name[k]);
            return 4;
        }
    }
    HIP_OK(hipMemcpy(h.data(), d.h, n * 2, hipMemcpyDeviceToHost));
    if (memcmp(h.data(), want.h.data(), n * 2) != 0) {
        fprintf(stderr, "%s: chunk %d fp16 param differs from the CPU restatement\n", what, chunk);
        return 4;
    }
    return 0;
}

void new_gradients(Lcg& rng, HostChunk& c, double scale)
{
    for (size_t i = 0; i < c.h.size(); ++i) c.h[i] = oracle_f32_to_f16((float)(rng.normal() * 1e-3 * scale));
}

}  // namespace

int main()
{
    int n_dev = 0;
    HIP_OK(hipGetDeviceCount(&n_dev));
    if (n_dev < 1) {
        fprintf(stderr, "no GPU\n");
        return 77;
    }
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    const int C = 3;
    const size_t n = 256 * 13 + 5;  // whole tiles and a ragged one
    const float lr = 1e-4f, b1 = 0.9f, b2 = 0.999f, eps = 1e-8f, wd = 0.01f;
    Lcg rng{12345};
    std::vector<HostChunk> host(C);
    std::vector<DeviceChunk> dev(C);
    ps_chunk table[C];
    for (int c = 0; c < C; ++c) {
        HostChunk& hc = host[c];
        hc.p.resize(n), hc.m.resize(n), hc.v.resize(n), hc.h.resize(n);
        for (size_t i = 0; i < n; ++i) {
            hc.p[i] = (float)(rng.normal() * 0.02);
            hc.m[i] = (float)(rng.normal() * 1e-4);
            hc.v[i] = (float)std::fabs(rng.normal() * 1e-6);
        }
        HIP_OK(hipMalloc((void**)&dev[c].p, n * 4));
        HIP_OK(hipMalloc((void**)&dev[c].m, n * 4));
        HIP_OK(hipMalloc((void**)&dev[c].v, n * 4));
        HIP_OK(hipMalloc((void**)&dev[c].h, n * 2));
        table[c].param_fp32 = dev[c].p;
        table[c].exp_avg = dev[c].m;
        table[c].exp_avg_sq = dev[c].v;
        table[c].param_fp16 = dev[c].h;
    }
    if (oracle_sizeof_state() > (int)sizeof(oracle_adam_opaque)) return 5;
    oracle_adam_opaque native;
    oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
    PS_OK(ps_adam_create(31, lr, b1, b2, eps, wd, 1, 0));

    // Every chunk holds one tensor: the reference makes one operator call per chunk and step, the first of them
    // for the whole of chunk 0.
    const ps_call_pattern calls = {C, 0, 0, n};

    // ---- host-decided steps with a static scale: t = 100 (cold), then 101 and 102 (the first call of each
    //      multiplies the running product, the later calls evaluate pow)
    const double scale = 4096.0;
    for (uint64_t step = 100; step < 103; ++step) {
        for (int c = 0; c < C; ++c) {
            new_gradients(rng, host[c], scale);
            if (upload(host[c], dev[c], n)) return 2;
        }
        PS_OK(ps_adam_step_chunks(31, step, lr, b1, b2, eps, wd, 1, table, C, n, nullptr, &calls, scale, stream));
        HIP_OK(hipStreamSynchronize(stream));
        for (int c = 0; c < C; ++c) {
            oracle_adam_advance(&native, step, b1, b2);  // one adam_update per tensor, same step number
            oracle_adam_set(&native, lr, eps, wd, 1);
            if (oracle_adam_span(&native, host[c].p.data(), host[c].h.data(), 1, host[c].m.data(), host[c].v.data(),
                                 n, (float)scale, 0) <= 0)
                return 5;
            oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
            if (int rc = compare(host[c], dev[c], n, "static step", c)) return rc;
        }
    }

    // ---- device-decided steps: probe, gated update, scale update; nothing is read back until the end
    ps_step_state* d_state = nullptr;
    HIP_OK(hipMalloc((void**)&d_state, sizeof(ps_step_state)));
    PS_OK(ps_state_init(d_state, 1024.0, 1, 2.0, 1, 3, 1.0, 1, 1, 0, b1, b2, stream));
    PS_OK(ps_adam_create(32, lr, b1, b2, eps, wd, 1, 0));
    oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
    double cur_scale = 1024.0;  // loss_scaler.py:158-182 with delayed_shift = 1
    int64_t cur_iter = 0, last_overflow = -1, adam_step = 0;
    for (int it = 0; it < 8; ++it) {
        const bool poison = it == 2 || it == 5;
        for (int c = 0; c < C; ++c) {
            new_gradients(rng, host[c], cur_scale);
            if (poison && c == it % C) host[c].h[n - 1] = 0x7C00;  // +inf in the last element
            if (upload(host[c], dev[c], n)) return 2;
        }
        PS_OK(ps_overflow_scan_chunks(table, C, n, nullptr, d_state, stream));
        PS_OK(ps_adam_step_chunks_gated(32, lr, eps, wd, 1, table, C, n, nullptr, &calls, d_state, stream));
        PS_OK(ps_scaler_update(d_state, PS_FLAG_FROM_DEVICE, NULL, 0, calls.n_calls, stream));
        HIP_OK(hipStreamSynchronize(stream));
        if (poison) {
            for (int c = 0; c < C; ++c) oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
            cur_scale = cur_scale / 2.0 > 1.0 ? cur_scale / 2.0 : 1.0;
            last_overflow = cur_iter;
        } else {
            adam_step += 1;
            for (int c = 0; c < C; ++c) {
                oracle_adam_advance(&native, (uint64_t)adam_step, b1, b2);
                oracle_adam_set(&native, lr, eps, wd, 1);
                if (oracle_adam_span(&native, host[c].p.data(), host[c].h.data(), 1, host[c].m.data(),
                                     host[c].v.data(), n, (float)cur_scale, 0) <= 0)
                    return 5;
                oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
            }
            if ((cur_iter - last_overflow) % 3 == 0) cur_scale *= 2.0;
        }
        cur_iter += 1;
        for (int c = 0; c < C; ++c)
            if (int rc = compare(host[c], dev[c], n, poison ? "skipped step" : "gated step", c)) return rc;
    }
    ps_step_state st;
    PS_OK(ps_state_read(d_state, &st, stream));
    if (st.cur_scale != cur_scale || st.cur_iter != cur_iter || st.adam_step != adam_step || st.skipped_steps != 2 ||
        st.overflow != 0) {
        fprintf(stderr, "step state: scale %g (want %g) iter %lld (%lld) step %lld (%lld) skipped %lld\n", st.cur_scale,
                cur_scale, (long long)st.cur_iter, (long long)cur_iter, (long long)st.adam_step, (long long)adam_step,
                (long long)st.skipped_steps);
        return 6;
    }
    PS_OK(ps_adam_destroy(31));
    PS_OK(ps_adam_destroy(32));

    // ---- host-resident chunk positions: fp32 param / m / v in pinned host memory, streamed through two staging
    //      slots; position 0 stays resident, position 1 keeps its fp16 payload in HBM, position 2 has it on the host
    struct PinnedChunk {
        float *p = nullptr, *m = nullptr, *v = nullptr;
        uint16_t* h = nullptr;  // pinned host memory, or NULL when the fp16 payload stays in HBM
    };
    PinnedChunk pinned[C];
    ps_chunk host_table[2], staging[2];
    for (int c = 1; c < C; ++c) {
        HIP_OK(hipHostMalloc((void**)&pinned[c].p, n * 4, hipHostMallocDefault));
        HIP_OK(hipHostMalloc((void**)&pinned[c].m, n * 4, hipHostMallocDefault));
        HIP_OK(hipHostMalloc((void**)&pinned[c].v, n * 4, hipHostMallocDefault));
        if (c == 2) HIP_OK(hipHostMalloc((void**)&pinned[c].h, n * 2, hipHostMallocDefault));
        host_table[c - 1].param_fp32 = pinned[c].p;
        host_table[c - 1].exp_avg = pinned[c].m;
        host_table[c - 1].exp_avg_sq = pinned[c].v;
        host_table[c - 1].param_fp16 = c == 2 ? pinned[c].h : dev[c].h;
    }
    for (int s = 0; s < 2; ++s) {
        HIP_OK(hipMalloc((void**)&staging[s].param_fp32, n * 4));
        HIP_OK(hipMalloc((void**)&staging[s].exp_avg, n * 4));
        HIP_OK(hipMalloc((void**)&staging[s].exp_avg_sq, n * 4));
        HIP_OK(hipMalloc((void**)&staging[s].param_fp16, n * 2));
    }
    PS_OK(ps_adam_create(33, lr, b1, b2, eps, wd, 1, 0));
    oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
    for (uint64_t step = 1; step < 4; ++step) {
        for (int c = 0; c < C; ++c) {
            new_gradients(rng, host[c], scale);
            if (c == 0) {
                if (upload(host[c], dev[c], n)) return 2;
            } else {
                memcpy(pinned[c].p, host[c].p.data(), n * 4);
                memcpy(pinned[c].m, host[c].m.data(), n * 4);
                memcpy(pinned[c].v, host[c].v.data(), n * 4);
                if (c == 2)
                    memcpy(pinned[c].h, host[c].h.data(), n * 2);
                else
                    HIP_OK(hipMemcpy(dev[c].h, host[c].h.data(), n * 2, hipMemcpyHostToDevice));
            }
        }
        PS_OK(ps_adam_step_hybrid(33, step, lr, b1, b2, eps, wd, 1, table, 1, host_table, 2, n, nullptr, staging, 2, &calls, scale,
                                  NULL, stream));
        HIP_OK(hipStreamSynchronize(stream));
        for (int c = 0; c < C; ++c) {
            oracle_adam_advance(&native, step, b1, b2);
            oracle_adam_set(&native, lr, eps, wd, 1);
            if (oracle_adam_span(&native, host[c].p.data(), host[c].h.data(), 1, host[c].m.data(), host[c].v.data(),
                                 n, (float)scale, 0) <= 0)
                return 5;
            oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
        }
        if (int rc = compare(host[0], dev[0], n, "hybrid step, resident", 0)) return rc;
        for (int c = 1; c < C; ++c) {
            bool same = memcmp(pinned[c].p, host[c].p.data(), n * 4) == 0 && memcmp(pinned[c].m, host[c].m.data(), n * 4) == 0 &&
                        memcmp(pinned[c].v, host[c].v.data(), n * 4) == 0;
            if (c == 2) {
                same = same && memcmp(pinned[c].h, host[c].h.data(), n * 2) == 0;
            } else {
                std::vector<uint16_t> h16(n);
                HIP_OK(hipMemcpy(h16.data(), dev[c].h, n * 2, hipMemcpyDeviceToHost));
                same = same && memcmp(h16.data(), host[c].h.data(), n * 2) == 0;
            }
            if (!same) {
                fprintf(stderr, "hybrid step %llu: host-resident chunk %d differs from the CPU restatement\n",
                        (unsigned long long)step, c);
                return 4;
            }
        }
    }
    // the probe over host-resident positions: an inf in the pinned fp16 payload must reach the device flag
    PS_OK(ps_state_init(d_state, 1024.0, 1, 2.0, 1, 1000, 1.0, 1, 1, 0, b1, b2, stream));
    pinned[2].h[n / 2] = 0xFC00;  // -inf
    PS_OK(ps_overflow_scan_host_chunks(host_table, 2, n, nullptr, staging, 2, d_state, stream));
    PS_OK(ps_state_read(d_state, &st, stream));
    if (st.overflow != 1) {
        fprintf(stderr, "the probe of host-resident chunks missed an inf\n");
        return 6;
    }
    PS_OK(ps_adam_destroy(33));

    // ---- tensor list: the chunks cut into tensors (two per chunk, the second at an odd element offset), listed in
    //      another order than the reference visits them and handed over in two calls under one call pattern; the
    //      reference's first call is the SECOND tensor of chunk 1
    {
        const size_t cut = 256 * 5 + 3;
        struct Span { int chunk; size_t off, len; };
        const Span order[6] = {{1, cut, n - cut}, {0, 0, cut}, {2, 0, cut}, {0, cut, n - cut}, {1, 0, cut}, {2, cut, n - cut}};  // reference order
        const int listed_a[2] = {3, 0}, listed_b[4] = {5, 4, 2, 1};  // indices into order[]; the first call is listed_a[1]
        PS_OK(ps_adam_create(34, lr, b1, b2, eps, wd, 1, 0));
        oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
        for (int c = 0; c < C; ++c)
            if (upload(host[c], dev[c], n)) return 2;
        for (uint64_t step = 1; step < 4; ++step) {
            for (int c = 0; c < C; ++c) {
                new_gradients(rng, host[c], scale);
                if (upload(host[c], dev[c], n)) return 2;
            }
            auto describe = [&](const int* idx, int count, ps_chunk* rows, size_t* lens) {
                for (int k = 0; k < count; ++k) {
                    const Span& t = order[idx[k]];
                    rows[k].param_fp32 = dev[t.chunk].p + t.off;
                    rows[k].exp_avg = dev[t.chunk].m + t.off;
                    rows[k].exp_avg_sq = dev[t.chunk].v + t.off;
                    rows[k].param_fp16 = dev[t.chunk].h + t.off;
                    lens[k] = t.len;
                }
            };
            ps_chunk rows_a[2], rows_b[4];
            size_t len_a[2], len_b[4];
            describe(listed_a, 2, rows_a, len_a);
            describe(listed_b, 4, rows_b, len_b);
            const ps_call_pattern first_here = {6, 1, 0, len_a[1]}, first_elsewhere = {6, 0, 0, 0};
            PS_OK(ps_adam_step_tensors(34, step, lr, b1, b2, eps, wd, 1, rows_a, len_a, 2, &first_here, scale, NULL, stream));
            PS_OK(ps_adam_step_tensors(34, step, lr, b1, b2, eps, wd, 1, rows_b, len_b, 4, &first_elsewhere, scale, NULL, stream));
            HIP_OK(hipStreamSynchronize(stream));
            for (const Span& t : order) {
                oracle_adam_advance(&native, step, b1, b2);
                oracle_adam_set(&native, lr, eps, wd, 1);
                HostChunk& hc = host[t.chunk];
                if (t.len && oracle_adam_span(&native, hc.p.data() + t.off, hc.h.data() + t.off, 1, hc.m.data() + t.off,
                                              hc.v.data() + t.off, t.len, (float)scale, 0) <= 0)
                    return 5;
            }
            for (int c = 0; c < C; ++c) {
                oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
                if (int rc = compare(host[c], dev[c], n, "tensor-list step", c)) return rc;
            }
        }
        PS_OK(ps_adam_destroy(34));
    }

    // ---- every tensor its own step number and hyper-parameters (ps_adam_step_tensors_each): six tensors, one of
    //      them standing three steps behind, one with another learning rate and no decay, one with other betas whose
    //      neighbour in the call order stands exactly one step ahead of it (that call multiplies in mid-step);
    //      host-decided first, then device-decided with a skipped step in between
    {
        const size_t cut = 256 * 4 + 77;
        struct Span { int chunk; size_t off, len; };
        const Span order[6] = {{2, cut, n - cut}, {0, 0, cut}, {0, cut, n - cut}, {1, 0, cut}, {1, cut, n - cut}, {2, 0, cut}};
        uint64_t steps_made[6] = {20, 20, 17, 20, 20, 21};   // state[p]["step"] before the next step
        const double lrs[6] = {1e-4, 1e-4, 1e-4, 5e-5, 1e-4, 1e-4}, wds[6] = {0.01, 0.01, 0.01, 0.0, 0.01, 0.01};
        const double be1[6] = {0.9, 0.9, 0.9, 0.9, 0.8, 0.8}, be2[6] = {0.999, 0.999, 0.999, 0.999, 0.99, 0.99};
        PS_OK(ps_adam_create(35, lr, b1, b2, eps, wd, 1, 0));
        oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
        ps_chunk rows[6];
        size_t lens[6];
        for (int k = 0; k < 6; ++k) {
            const Span& t = order[k];
            rows[k].param_fp32 = dev[t.chunk].p + t.off;
            rows[k].exp_avg = dev[t.chunk].m + t.off;
            rows[k].exp_avg_sq = dev[t.chunk].v + t.off;
            rows[k].param_fp16 = dev[t.chunk].h + t.off;
            lens[k] = t.len;
        }
        auto oracle_calls = [&](double loss_scale) -> int {
            for (int k = 0; k < 6; ++k) {
                const Span& t = order[k];
                steps_made[k] += 1;
                oracle_adam_advance(&native, steps_made[k], (float)be1[k], (float)be2[k]);
                oracle_adam_set(&native, (float)lrs[k], eps, (float)wds[k], 1);
                HostChunk& hc = host[t.chunk];
                if (oracle_adam_span(&native, hc.p.data() + t.off, hc.h.data() + t.off, 1, hc.m.data() + t.off,
                                     hc.v.data() + t.off, t.len, (float)loss_scale, 0) <= 0)
                    return 5;
            }
            for (int c = 0; c < C; ++c) oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
            return 0;
        };
        ps_tensor_call each[6];
        for (int it = 0; it < 2; ++it) {  // host-decided
            for (int c = 0; c < C; ++c) {
                new_gradients(rng, host[c], scale);
                if (upload(host[c], dev[c], n)) return 2;
            }
            for (int k = 0; k < 6; ++k)
                each[k] = ps_tensor_call{lrs[k], be1[k], be2[k], eps, wds[k], (int64_t)steps_made[k] + 1, -1, 0};
            PS_OK(ps_adam_step_tensors_each(35, 1, rows, lens, each, 6, scale, NULL, NULL, 0, stream));
            HIP_OK(hipStreamSynchronize(stream));
            if (int rc = oracle_calls(scale)) return rc;
            for (int c = 0; c < C; ++c)
                if (int rc = compare(host[c], dev[c], n, "per-tensor step, host-decided", c)) return rc;
        }
        // device-decided: the device's counter stands at tensor 0's count; every tensor says how far from it it stands
        void* d_work = nullptr;
        const size_t work_bytes = ps_tensors_each_workspace_bytes(6);
        HIP_OK(hipMalloc(&d_work, work_bytes));
        PS_OK(ps_state_init(d_state, 256.0, 1, 2.0, 1, 1000, 1.0, 1, 1, 0, b1, b2, stream));
        // the operator object goes on running (fresh_operator = 0 would need the device to hold it; this library object is
        // the host's, so the device starts from a fresh one and so does the restatement)
        PS_OK(ps_state_seed_step(d_state, (int64_t)steps_made[0], b1, b2, 1, stream));
        oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
        double dyn_scale = 256.0;
        for (int it = 0; it < 3; ++it) {
            const bool poison = it == 1;
            for (int c = 0; c < C; ++c) {
                new_gradients(rng, host[c], dyn_scale);
                if (poison && c == 1) host[c].h[7] = 0x7E00;  // nan
                if (upload(host[c], dev[c], n)) return 2;
            }
            for (int k = 0; k < 6; ++k)
                each[k] = ps_tensor_call{lrs[k], be1[k], be2[k], eps, wds[k], (int64_t)steps_made[k] - (int64_t)steps_made[0], -1, 0};
            PS_OK(ps_overflow_scan_chunks(table, C, n, nullptr, d_state, stream));
            PS_OK(ps_adam_step_tensors_each(35, 1, rows, lens, each, 6, -1.0, d_state, d_work, work_bytes, stream));
            PS_OK(ps_scaler_update(d_state, PS_FLAG_FROM_DEVICE, NULL, 0, 6, stream));
            HIP_OK(hipStreamSynchronize(stream));
            if (poison) {
                for (int c = 0; c < C; ++c) oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
                dyn_scale /= 2.0;
            } else if (int rc = oracle_calls(dyn_scale)) {
                return rc;
            }
            for (int c = 0; c < C; ++c)
                if (int rc = compare(host[c], dev[c], n, poison ? "per-tensor step, skipped" : "per-tensor step, device-decided", c)) return rc;
        }
        PS_OK(ps_state_read(d_state, &st, stream));
        if (st.adam_step != (int64_t)steps_made[0] || st.cur_scale != dyn_scale || st.pending_operator_step != 0) {
            fprintf(stderr, "per-tensor steps: device counter %lld (want %llu), scale %g (want %g)\n", (long long)st.adam_step,
                    (unsigned long long)steps_made[0], st.cur_scale, dyn_scale);
            return 6;
        }
        HIP_OK(hipFree(d_work));
        PS_OK(ps_adam_destroy(35));
    }

    // ---- a tensor with a binary32 gradient and no fp16 copy (PS_TENSOR_GRAD_F32: what the reference's loop does for
    //      parameters PyTorch manages itself) as the step's FIRST operator call, in front of two whole chunks
    {
        const size_t nf = 256 * 5 + 19;
        std::vector<float> fp(nf), fm(nf, 0.0f), fv(nf, 0.0f), fg(nf);
        for (size_t i = 0; i < nf; ++i) fp[i] = (float)(rng.normal() * 0.02);
        float *dp = nullptr, *dm = nullptr, *dv = nullptr, *dg = nullptr;
        HIP_OK(hipMalloc(&dp, nf * 4));
        HIP_OK(hipMalloc(&dm, nf * 4));
        HIP_OK(hipMalloc(&dv, nf * 4));
        HIP_OK(hipMalloc(&dg, nf * 4));
        HIP_OK(hipMemcpy(dp, fp.data(), nf * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dm, fm.data(), nf * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dv, fv.data(), nf * 4, hipMemcpyHostToDevice));
        PS_OK(ps_adam_create(36, lr, b1, b2, eps, wd, 1, 0));
        oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
        ps_chunk rows[3];
        size_t lens[3] = {nf, n, n};
        rows[0].param_fp32 = dp, rows[0].exp_avg = dm, rows[0].exp_avg_sq = dv;
        rows[0].param_fp16 = reinterpret_cast<uint16_t*>(dg);  // the address of the binary32 gradient
        for (int c = 0; c < 2; ++c)
            rows[1 + c].param_fp32 = dev[c].p, rows[1 + c].exp_avg = dev[c].m, rows[1 + c].exp_avg_sq = dev[c].v,
                     rows[1 + c].param_fp16 = dev[c].h;
        ps_tensor_call each[3];
        for (uint64_t step = 1; step <= 3; ++step) {
            for (size_t i = 0; i < nf; ++i) fg[i] = (float)(rng.normal() * 1e-3 * scale);
            HIP_OK(hipMemcpy(dg, fg.data(), nf * 4, hipMemcpyHostToDevice));
            for (int c = 0; c < 2; ++c) {
                new_gradients(rng, host[c], scale);
                if (upload(host[c], dev[c], n)) return 2;
            }
            for (int k = 0; k < 3; ++k)
                each[k] = ps_tensor_call{lr, b1, b2, eps, wd, (int64_t)step, -1, k == 0 ? PS_TENSOR_GRAD_F32 : 0};
            PS_OK(ps_adam_step_tensors_each(36, 1, rows, lens, each, 3, scale, NULL, NULL, 0, stream));
            HIP_OK(hipStreamSynchronize(stream));
            oracle_adam_advance(&native, step, b1, b2);
            oracle_adam_set(&native, lr, eps, wd, 1);
            if (oracle_adam_span(&native, fp.data(), fg.data(), 0, fm.data(), fv.data(), nf, (float)scale, 0) <= 0) return 5;
            for (int c = 0; c < 2; ++c) {
                oracle_adam_advance(&native, step, b1, b2);
                oracle_adam_set(&native, lr, eps, wd, 1);
                if (oracle_adam_span(&native, host[c].p.data(), host[c].h.data(), 1, host[c].m.data(), host[c].v.data(), n,
                                     (float)scale, 0) <= 0)
                    return 5;
                oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
                if (int rc = compare(host[c], dev[c], n, "step with a binary32-gradient tensor", c)) return rc;
            }
            std::vector<float> back(nf);
            const float* src[4] = {dp, dm, dv, dg};
            const std::vector<float>* want[4] = {&fp, &fm, &fv, &fg};
            for (int k = 0; k < 4; ++k) {
                HIP_OK(hipMemcpy(back.data(), src[k], nf * 4, hipMemcpyDeviceToHost));
                if (memcmp(back.data(), want[k]->data(), nf * 4) != 0) {
                    fprintf(stderr, "binary32-gradient tensor: array %d differs from the CPU restatement at step %llu\n", k,
                            (unsigned long long)step);
                    return 4;
                }
            }
        }
        HIP_OK(hipFree(dp));
        HIP_OK(hipFree(dm));
        HIP_OK(hipFree(dv));
        HIP_OK(hipFree(dg));
        PS_OK(ps_adam_destroy(36));
    }

    // ---- a chunk list whose last chunk ends in zero padding: the step leaves the padding alone, same bits
    {
        const size_t used_last = 256 * 6 + 9;
        HostChunk& last = host[C - 1];
        for (size_t i = used_last; i < n; ++i) last.p[i] = last.m[i] = last.v[i] = 0.0f, last.h[i] = 0;
        PS_OK(ps_adam_create(36, lr, b1, b2, eps, wd, 1, 0));
        oracle_adam_init(&native, lr, b1, b2, eps, wd, 1);
        const size_t used[C] = {n, n, used_last};
        for (uint64_t step = 1; step < 3; ++step) {
            for (int c = 0; c < C; ++c) {
                new_gradients(rng, host[c], scale);
                if (c == C - 1)
                    for (size_t i = used_last; i < n; ++i) host[c].h[i] = 0;
                if (upload(host[c], dev[c], n)) return 2;
            }
            PS_OK(ps_adam_step_chunks(36, step, lr, b1, b2, eps, wd, 1, table, C, n, used, &calls, scale, stream));
            HIP_OK(hipStreamSynchronize(stream));
            for (int c = 0; c < C; ++c) {
                oracle_adam_advance(&native, step, b1, b2);
                oracle_adam_set(&native, lr, eps, wd, 1);
                if (oracle_adam_span(&native, host[c].p.data(), host[c].h.data(), 1, host[c].m.data(), host[c].v.data(), n,
                                     (float)scale, 0) <= 0)  // the restatement updates every slot, padding included
                    return 5;
                oracle_cast_f32_to_f16(host[c].p.data(), host[c].h.data(), n);
                if (int rc = compare(host[c], dev[c], n, "step over a padded chunk list", c)) return rc;
            }
        }
        PS_OK(ps_adam_destroy(36));
    }

    // ---- the probe that allocates nothing: same answer as the probe with a caller-side state
    {
        uint32_t* d_flag = nullptr;
        HIP_OK(hipMalloc((void**)&d_flag, sizeof(uint32_t)));
        HIP_OK(hipMemsetAsync(d_flag, 0, sizeof(uint32_t), stream));
        uint32_t flag = 7;
        PS_OK(ps_overflow_scan_chunks_noalloc(table, C, n, d_flag, stream));
        HIP_OK(hipMemcpyAsync(&flag, d_flag, sizeof(flag), hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        if (flag != 0) {
            fprintf(stderr, "the allocation-free probe saw an inf / nan in finite payloads\n");
            return 7;
        }
        const uint16_t nan16 = 0x7E00;
        HIP_OK(hipMemcpyAsync(dev[C - 1].h + (n - 1), &nan16, sizeof(nan16), hipMemcpyHostToDevice, stream));
        PS_OK(ps_overflow_scan_chunks_noalloc(table, C, n, d_flag, stream));
        HIP_OK(hipMemcpyAsync(&flag, d_flag, sizeof(flag), hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        if (flag != 1) {
            fprintf(stderr, "the allocation-free probe missed a nan in the last element of the last chunk\n");
            return 7;
        }
        HIP_OK(hipFree(d_flag));
    }
    printf("c abi gpu check ok: 3 host-decided and 8 device-decided steps (2 skipped), 3 steps with host-resident chunks, "
           "3 tensor-list steps in two calls each, 5 steps with per-tensor step numbers and hyper-parameters, 3 with a binary32-gradient tensor as the first call, 2 over a padded list, "
           "the allocation-free probe, over %d x %zu elements\n", C, n);
    return 0;
}
