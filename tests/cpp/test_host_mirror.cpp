// GPU test program (run by tests/test_gpu_host_mirror.py): drives the C++ mirror of the reference's
// ml.Backend / Context / Tensor interface and checks every Mulmat against the CPU oracle.
// Links libmi_qmm.so (the product) and oracle/libggml_ref.so (the checker; test infrastructure).
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "../../ollama_amd/host/ml_backend.hpp"
#include "../../oracle/ggml_ref.h"

using namespace ollama_amd;

static std::vector<float> randn(size_t n, float std, unsigned seed) {
    std::mt19937 g(seed);
    std::normal_distribution<float> d(0.f, std);
    std::vector<float> v(n);
    for (auto &x : v) x = d(g);
    return v;
}

static double rel_err(const std::vector<float> &y, const std::vector<float> &ref) {
    double ss = 0;
    for (float r : ref) ss += (double)r * r;
    const double floor_ = 1e-2 * std::sqrt(ss / ref.size());
    double worst = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        const double den = std::fmax(std::fabs((double)ref[i]), floor_);
        worst = std::fmax(worst, std::fabs((double)y[i] - ref[i]) / (den > 0 ? den : 1));
    }
    return worst;
}

int main() {
    try {
        Backend backend(0);
        struct Spec { const char *name; int type; int64_t k, m; };
        const Spec specs[] = {{"blk.0.attn_q.weight", MI_QMM_TYPE_Q4_K, 1024, 512}, {"blk.0.attn_k.weight", MI_QMM_TYPE_Q4_K, 1024, 128},
                              {"blk.0.ffn_down.weight", MI_QMM_TYPE_Q6_K, 1024, 256}, {"output.weight", MI_QMM_TYPE_Q8_0, 1024, 300},
                              {"legacy.weight", MI_QMM_TYPE_Q4_0, 1024, 64}};
        std::vector<std::vector<uint8_t>> raws;
        for (const Spec &s : specs) {
            auto wf = randn((size_t)(s.k * s.m), 0.02f, 17 + (unsigned)s.m);
            std::vector<uint8_t> raw((size_t)(ref_row_size(s.type, s.k) * s.m));
            if (ref_quantize(s.type, wf.data(), raw.data(), s.k, s.m, 4) != 0) { printf("FAIL: encode %s\n", s.name); return 1; }
            backend.Load(s.name, s.type, s.k, s.m, raw.data());
            raws.push_back(std::move(raw));
        }
        if (backend.Get("missing.weight") != nullptr) { printf("FAIL: Get of an unknown name\n"); return 1; }
        int failures = 0;
        for (int64_t n : {1, 3, 40}) {  // decode, skinny, prefill-sized batch
            auto ctx = backend.NewContext();
            auto xv = randn((size_t)(1024 * n), 1.0f, 99 + (unsigned)n);
            auto x = ctx->FromFloats(xv, {1024, n});
            std::vector<std::shared_ptr<Tensor>> outs;
            for (const Spec &s : specs) outs.push_back(backend.Get(s.name)->Mulmat(*ctx, x));
            ctx->Compute();
            for (size_t i = 0; i < outs.size(); i++) {
                const Spec &s = specs[i];
                std::vector<float> ref((size_t)(s.m * n));
                if (ref_mul_mat(s.type, raws[i].data(), s.k, s.m, xv.data(), n, ref.data(), nullptr, 4) != 0) return 1;
                const double e = rel_err(outs[i]->Floats(), ref);
                const bool shape_ok = outs[i]->Dim(0) == s.m && outs[i]->Dim(1) == n;
                printf("%-24s n=%-3lld rel err %.2e %s\n", s.name, (long long)n, e, (e <= 1e-3 && shape_ok) ? "ok" : "FAIL");
                if (!(e <= 1e-3) || !shape_ok) failures++;
            }
            ctx->Close();
        }
        // error behaviour: mismatched inner dimension throws, like the Go interface panics
        bool threw = false;
        try {
            auto ctx = backend.NewContext();
            backend.Get("output.weight")->Mulmat(*ctx, ctx->FromFloats(std::vector<float>(512), {512, 1}));
        } catch (const Error &) { threw = true; }
        if (!threw) { printf("FAIL: dimension mismatch did not throw\n"); failures++; }
        // the same weights from a GGUF file: written here byte by byte (header, one key-value, tensor
        // infos, padding to 32, data), loaded through LoadFile, results must equal the in-memory ones
        {
            std::string bytes = "GGUF";
            auto put = [&](const void *p, size_t n) { bytes.append(static_cast<const char *>(p), n); };
            auto put_u32 = [&](uint32_t v) { put(&v, 4); };
            auto put_u64 = [&](uint64_t v) { put(&v, 8); };
            auto put_str = [&](const std::string &v) { put_u64(v.size()); put(v.data(), v.size()); };
            put_u32(3); put_u64(2); put_u64(1);
            put_str("general.architecture"); put_u32(8); put_str("llama");
            uint64_t off = 0;
            std::vector<uint64_t> offs;
            for (int i = 0; i < 2; i++) {
                put_str(specs[i].name); put_u32(2); put_u64((uint64_t)specs[i].k); put_u64((uint64_t)specs[i].m);
                put_u32((uint32_t)specs[i].type); put_u64(off);
                offs.push_back(off);
                off += raws[i].size();
                off += (32 - off % 32) % 32;
            }
            bytes.append((32 - bytes.size() % 32) % 32, '\0');
            const size_t base = bytes.size();
            bytes.resize(base + off, '\0');
            for (int i = 0; i < 2; i++) memcpy(&bytes[base + offs[i]], raws[i].data(), raws[i].size());
            const std::string path = "/tmp/mi_qmm_host_mirror_test.gguf";
            FILE *fp = fopen(path.c_str(), "wb");
            if (!fp || fwrite(bytes.data(), 1, bytes.size(), fp) != bytes.size()) { printf("FAIL: cannot write %s\n", path.c_str()); return 1; }
            fclose(fp);
            Backend from_file(0);
            const int loaded = from_file.LoadFile(path);
            remove(path.c_str());
            if (loaded != 2) { printf("FAIL: LoadFile loaded %d tensors, want 2\n", loaded); failures++; }
            auto xv = randn(1024 * 2, 1.0f, 5);
            for (int i = 0; i < 2 && loaded == 2; i++) {
                auto c1 = backend.NewContext();
                auto c2 = from_file.NewContext();
                auto y1 = backend.Get(specs[i].name)->Mulmat(*c1, c1->FromFloats(xv, {1024, 2}));
                auto y2 = from_file.Get(specs[i].name)->Mulmat(*c2, c2->FromFloats(xv, {1024, 2}));
                c1->Compute();
                c2->Compute();
                const bool same = y1->Floats() == y2->Floats();
                printf("%-24s from file %s\n", specs[i].name, same ? "ok" : "FAIL");
                if (!same) failures++;
            }
            from_file.Close();
        }
        // expert-indexed product: a stack of 5 experts, 3 used per token, one activation row per token
        {
            const int64_t k = 1024, m = 96, n_expert = 5, n_used = 3;
            auto wf = randn((size_t)(k * m * n_expert), 0.02f, 1234);
            std::vector<uint8_t> raw((size_t)(ref_row_size(MI_QMM_TYPE_Q4_K, k) * m * n_expert));
            if (ref_quantize(MI_QMM_TYPE_Q4_K, wf.data(), raw.data(), k, m * n_expert, 4) != 0) return 1;
            backend.LoadExperts("blk.0.ffn_up_exps.weight", MI_QMM_TYPE_Q4_K, k, m, n_expert, raw.data());
            for (int64_t tokens : {1, 11}) {
                auto ctx = backend.NewContext();
                auto xv = randn((size_t)(k * tokens), 1.0f, 77 + (unsigned)tokens);
                std::vector<int32_t> idv;
                for (int64_t t = 0; t < tokens; t++)
                    for (int64_t i = 0; i < n_used; i++) idv.push_back((int32_t)((t * 2 + i * 3) % n_expert));
                auto y = backend.Get("blk.0.ffn_up_exps.weight")
                             ->MulmatID(*ctx, ctx->FromFloats(xv, {k, 1, tokens}), ctx->FromInts(idv, {n_used, tokens}));
                ctx->Compute();
                std::vector<float> ref((size_t)(m * n_used * tokens));
                if (ref_mul_mat_id(MI_QMM_TYPE_Q4_K, raw.data(), k, m, n_expert, xv.data(), 1, idv.data(), n_used, tokens,
                                   ref.data()) != 0) return 1;
                const double e = rel_err(y->Floats(), ref);
                const bool shape_ok = y->Dim(0) == m && y->Dim(1) == n_used && y->Dim(2) == tokens;
                printf("%-24s T=%-3lld rel err %.2e %s\n", "ffn_up_exps MulmatID", (long long)tokens, e,
                       (e <= 1e-3 && shape_ok) ? "ok" : "FAIL");
                if (!(e <= 1e-3) || !shape_ok) failures++;
                ctx->Close();
            }
            // the expert block's last step: silu(gate) * up inside the down experts' quantization
            for (int64_t tokens : {1, 5}) {  // one token: gate, up and the gating are one call
                const int64_t f = m;   // the stack above as gate and up: [k -> m]; a down stack [m -> 64]
                auto wf2 = randn((size_t)(f * 64 * n_expert), 0.02f, 4321);
                std::vector<uint8_t> rawd((size_t)(ref_row_size(MI_QMM_TYPE_Q8_0, f) * 64 * n_expert));
                if (ref_quantize(MI_QMM_TYPE_Q8_0, wf2.data(), rawd.data(), f, 64 * n_expert, 4) != 0) return 1;
                backend.LoadExperts("blk.0.ffn_down_exps.weight", MI_QMM_TYPE_Q8_0, f, 64, n_expert, rawd.data());
                auto ctx = backend.NewContext();
                auto xv = randn((size_t)(k * tokens), 1.0f, 901);
                std::vector<int32_t> idv;
                for (int64_t t = 0; t < tokens; t++)
                    for (int64_t i = 0; i < n_used; i++) idv.push_back((int32_t)((t + i * 2) % n_expert));
                auto ids = ctx->FromInts(idv, {n_used, tokens});
                auto x = ctx->FromFloats(xv, {k, 1, tokens});
                auto g = backend.Get("blk.0.ffn_up_exps.weight")->MulmatID(*ctx, x, ids);
                auto u = backend.Get("blk.0.ffn_up_exps.weight")->MulmatID(*ctx, x, ids);
                auto act = g->SILU(*ctx, u);
                auto out = backend.Get("blk.0.ffn_down_exps.weight")->MulmatID(*ctx, act, ids);
                ctx->Compute();
                bool lazy_g = false;
                try { g->Floats(); } catch (const Error &) { lazy_g = true; }
                if (lazy_g != (tokens == 1)) { printf("FAIL: expert gate materialized=%d at T=%lld\n", !lazy_g, (long long)tokens); failures++; }
                std::vector<float> gv((size_t)(f * n_used * tokens)), uv(gv.size()), av(gv.size()), ref((size_t)(64 * n_used * tokens));
                if (ref_mul_mat_id(MI_QMM_TYPE_Q4_K, raw.data(), k, m, n_expert, xv.data(), 1, idv.data(), n_used, tokens, gv.data()) != 0) return 1;
                uv = gv;  // gate and up are the same stack here
                ref_swiglu(gv.data(), uv.data(), (int64_t)av.size(), av.data());
                if (ref_mul_mat_id(MI_QMM_TYPE_Q8_0, rawd.data(), f, 64, n_expert, av.data(), n_used, idv.data(), n_used, tokens,
                                   ref.data()) != 0) return 1;
                const double e = rel_err(out->Floats(), ref);
                printf("%-24s T=%-3lld rel err %.2e %s\n", "expert block, SILU fused", (long long)tokens, e, e <= 2e-3 ? "ok" : "FAIL");
                if (!(e <= 2e-3)) failures++;
                ctx->Close();
            }
            bool threw_id = false;
            try {
                auto ctx = backend.NewContext();
                backend.Get("blk.0.ffn_up_exps.weight")
                    ->MulmatID(*ctx, ctx->FromFloats(std::vector<float>(k), {k, 1, 1}), ctx->FromInts({5}, {1, 1}));
                ctx->Compute();
            } catch (const Error &) { threw_id = true; }
            if (!threw_id) { printf("FAIL: an expert id outside the stack did not throw\n"); failures++; }
        }
        // feed-forward block with its producers: x -> RMSNorm -> gate, up -> SILU(gate, up) -> down
        {
            const int64_t k = 1024, f = 768;
            struct M { const char *name; int type; int64_t kk, m; };
            const M mats[] = {{"blk.1.ffn_gate.weight", MI_QMM_TYPE_Q4_K, k, f}, {"blk.1.ffn_up.weight", MI_QMM_TYPE_Q4_K, k, f},
                              {"blk.1.ffn_down.weight", MI_QMM_TYPE_Q6_K, f, k}};
            std::vector<std::vector<uint8_t>> fr;
            for (const M &m : mats) {
                auto wf = randn((size_t)(m.kk * m.m), 0.05f, 300 + (unsigned)fr.size());
                std::vector<uint8_t> raw((size_t)(ref_row_size(m.type, m.kk) * m.m));
                if (ref_quantize(m.type, wf.data(), raw.data(), m.kk, m.m, 4) != 0) return 1;
                backend.Load(m.name, m.type, m.kk, m.m, raw.data());
                fr.push_back(std::move(raw));
            }
            auto g = randn((size_t)k, 0.1f, 55);
            for (auto &v : g) v += 1.0f;
            backend.Load("blk.1.ffn_norm.weight", MI_QMM_TYPE_F32, k, 1, g.data());
            for (int64_t n : {1, 5, 40}) {
                auto xv = randn((size_t)(k * n), 1.0f, 500 + (unsigned)n);
                std::vector<float> outs[2];
                for (int pass = 0; pass < 2; pass++) {  // 0: producers fused into the products; 1: materialized
                    auto ctx = backend.NewContext();
                    auto x = ctx->FromFloats(xv, {k, n});
                    auto h = x->RMSNorm(*ctx, backend.Get("blk.1.ffn_norm.weight"), 1e-5f);
                    auto gate = backend.Get("blk.1.ffn_gate.weight")->Mulmat(*ctx, h);
                    auto up = backend.Get("blk.1.ffn_up.weight")->Mulmat(*ctx, h);
                    auto act = gate->SILU(*ctx, up);
                    auto out = backend.Get("blk.1.ffn_down.weight")->Mulmat(*ctx, act);
                    if (pass == 0) ctx->Compute(); else ctx->Compute({h, gate, up, act});
                    bool lazy = false, lazy_gate = false;
                    try { h->Floats(); } catch (const Error &) { lazy = true; }
                    try { gate->Floats(); } catch (const Error &) { lazy_gate = true; }
                    if (lazy != (pass == 0) || lazy_gate != (pass == 0 && n == 1)) {  // one row: gate and up absorbed too
                        printf("FAIL: norm materialized=%d gate materialized=%d in pass %d\n", !lazy, !lazy_gate, pass);
                        failures++;
                    }
                    outs[pass] = out->Floats();
                    if (pass == 1) {
                        std::vector<float> hv(xv.size()), gv((size_t)(f * n)), uv((size_t)(f * n)), av((size_t)(f * n)), ref((size_t)(k * n));
                        ref_rms_norm(xv.data(), g.data(), 1e-5f, k, n, hv.data());
                        ref_mul_mat(MI_QMM_TYPE_Q4_K, fr[0].data(), k, f, hv.data(), n, gv.data(), nullptr, 4);
                        ref_mul_mat(MI_QMM_TYPE_Q4_K, fr[1].data(), k, f, hv.data(), n, uv.data(), nullptr, 4);
                        const double eg = rel_err(gate->Floats(), gv);
                        // the last step alone: the oracle on the GPU's own gate / up values
                        ref_swiglu(gate->Floats().data(), up->Floats().data(), f * n, av.data());
                        ref_mul_mat(MI_QMM_TYPE_Q6_K, fr[2].data(), f, k, av.data(), n, ref.data(), nullptr, 4);
                        const double e = rel_err(out->Floats(), ref);
                        printf("%-24s N=%-3lld rel err gate %.2e down %.2e %s\n", "ffn block with producers", (long long)n, eg, e,
                               (eg <= 1e-3 && e <= 1e-3) ? "ok" : "FAIL");
                        if (!(eg <= 1e-3) || !(e <= 1e-3)) failures++;
                    }
                    ctx->Close();
                }
                if (outs[0] != outs[1]) { printf("FAIL: fused and materialized producers differ at N=%lld\n", (long long)n); failures++; }
            }
            {   // the bare activation SILU(ctx): an f32 node of its own
                auto ctx = backend.NewContext();
                std::vector<float> v(k);
                for (int64_t i = 0; i < k; i++) v[i] = 0.01f * (float)(i % 400) - 2.f;
                auto bare = ctx->FromFloats(v, {k, 1})->SILU(*ctx);
                ctx->Compute({bare});
                double worst = 0;
                for (int64_t i = 0; i < k; i++) {
                    const double want = (double)v[i] / (1.0 + std::exp(-(double)v[i]));
                    worst = std::max(worst, std::fabs((double)bare->Floats()[i] - want));
                }
                if (!(worst <= 1e-6)) { printf("FAIL: bare SILU off by %.3g\n", worst); failures++; }
                ctx->Close();
            }
        }
        backend.Close();
        printf(failures ? "host mirror: %d FAILURES\n" : "host mirror: all ok\n", failures);
        return failures ? 1 : 0;
    } catch (const Error &e) {
        printf("FAIL: mi_qmm error %d: %s\n", e.code, e.what());
        return 2;
    }
}
