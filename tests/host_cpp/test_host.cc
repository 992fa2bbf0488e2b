// The reference's own GPU tests for this path, restated in C++ against the host mirror
// (saetta-macqwen_amd/host/saetta.hpp) with the CPU oracle as the other side:
//   tests/kv_quant.rs   prefill_rows_match_cpu, decode_row_matches_cpu, dequantize_matches_cpu
//   tests/attention.rs  quantized_matches_cpu
//   tests/attention_prefill.rs  (one shape) for attention_prefill::encode and attention_gemm::AttGemm::encode
// Exit code 0 = all passed.  Run by tests/test_gpu_host_cpp.py on a GPU box.
#include <cstdio>
#include <cstdlib>

#include "../../saetta-macqwen_amd/host/saetta.hpp"

extern "C" {  // oracle/saetta_oracle.c (the checker)
int orc_quantize(const float *x, size_t n, int bits, uint32_t *data, uint16_t *scales, uint16_t *biases);
int orc_dequantize(const uint32_t *data, const uint16_t *scales, const uint16_t *biases, size_t groups, int bits, float *out);
uint16_t orc_f32_to_f16(float f);
void orc_noise(float *out, size_t n, uint64_t seed);
void orc_quant_rows(float *out, size_t tokens, size_t values);
int orc_attention_f64(const float *q, const float *k, const float *v, const float *q_and_gate, size_t len, size_t heads,
                      size_t kv_heads, size_t dim, double *out, int threads);
int orc_prefill(const float *q, const float *keys, const float *values, size_t pos, size_t tokens, size_t heads,
                size_t kv_heads, size_t dim, const float *q_and_gate, float *out, int threads);
}

using namespace saetta;
using kv_quant::KvBits;
using kv_quant::QuantRows;

static int failures = 0;
#define EXPECT(cond, ...)                 \
    do {                                  \
        if (!(cond)) {                    \
            failures++;                   \
            std::printf("FAIL: " __VA_ARGS__); \
            std::printf("\n");            \
        }                                 \
    } while (0)

constexpr size_t VALUES = 2 * 256, HEADS = 16, KV = 2, DIM = 256;

static void compare(const QuantRows &rows, const std::vector<float> &x, size_t from_token, KvBits bits) {
    const int b = int(kv_quant::bits(bits));
    const size_t groups = x.size() / 64, first = from_token * rows.per_token, words = kv_quant::words_per_group(bits);
    auto data = gpu::contents<uint32_t>(rows.data, groups * words, first * words * 4);
    auto scales = gpu::contents<uint16_t>(rows.scales, groups, first * 2);
    auto biases = gpu::contents<uint16_t>(rows.biases, groups, first * 2);
    std::vector<uint32_t> wd(groups * words);
    std::vector<uint16_t> ws(groups), wz(groups);
    orc_quantize(x.data(), x.size(), b, wd.data(), ws.data(), wz.data());
    EXPECT(scales == ws, "%d-bit scales", b);
    EXPECT(biases == wz, "%d-bit biases", b);
    size_t off = 0;
    for (size_t i = 0; i < wd.size(); i++) off += data[i] != wd[i];
    EXPECT(off == 0, "%d-bit: %zu code words differ", b, off);
}

int main() {
    gpu::Gpu gpu;
    for (KvBits bits : {KvBits::Eight, KvBits::Four}) {
        {  // prefill_rows_match_cpu
            const size_t tokens = 37;
            QuantRows cache(gpu, bits, VALUES, 64);
            std::vector<float> x(tokens * VALUES);
            orc_quant_rows(x.data(), tokens, VALUES);
            View xb(gpu.buffer_from(x));
            cache.encode(gpu, xb, 5, tokens);
            gpu.sync();
            compare(cache, x, 5, bits);
        }
        {  // decode_row_matches_cpu
            QuantRows cache(gpu, bits, VALUES, 64);
            std::vector<float> x(VALUES);
            orc_quant_rows(x.data(), 1, VALUES);
            View xb(gpu.buffer_from(x));
            plan::Plan plan(gpu);
            cache.record(plan, xb);
            auto built = plan.build();
            plan.set_params(plan::token_params(0, 41));
            built.run(gpu);
            compare(cache, x, 41, bits);
            // serial == replay (tests/plan.rs:27-45), and the rest of Plan and Built
            QuantRows second(gpu, bits, VALUES, 64);
            second.record(plan, xb);
            EXPECT(plan.len() == 2 && !plan.is_empty() && plan::Plan(gpu).is_empty(), "Plan::len");
            const auto kernels = plan.kernels();
            EXPECT(kernels.size() == 1 && kernels[0].second == 2 && kernels[0].first.rfind("kv_quantize", 0) == 0, "Plan::kernels");
            plan.set_params(plan::token_params(0, 7));
            EXPECT(plan.run_serial() > 0.0, "Plan::run_serial");
            compare(second, x, 7, bits);
            auto graph = plan.build(true);
            plan.set_params(plan::token_params(0, 50));
            const auto timed = graph.run_timed(gpu);
            EXPECT(timed.first > 0.0 && timed.second > 0.0 && timed.second <= timed.first, "Built::run_timed %g %g", timed.first, timed.second);
            compare(second, x, 50, bits);
            compare(cache, x, 50, bits);
            plan.set_params(plan::token_params(0, 60));
            graph.commit(gpu).wait();
            compare(second, x, 60, bits);
            const View c = plan.constant(std::vector<float>{1.5f, 2.5f});
            EXPECT(gpu::contents<float>(c.buffer, 2) == (std::vector<float>{1.5f, 2.5f}), "Plan::constant");
            // set_params is ordered by the stream without a wait: many positions back to back, the last one counts
            for (uint32_t pos = 0; pos < 40; pos++) {
                plan.set_params(plan::token_params(0, pos % 60));
                graph.commit(gpu);
            }
            gpu.sync();
            compare(second, x, 39, bits);
            // an op that throws while the plan is captured leaves the stream usable
            plan::Plan bad(gpu);
            second.record(bad, xb);
            bad.op("throws", [](hipStream_t) { throw std::runtime_error("refused"); });
            bool thrown = false;
            try {
                bad.build(true);
            } catch (const std::runtime_error &) {
                thrown = true;
            }
            EXPECT(thrown, "an op's exception comes out of Plan::build");
            plan.set_params(plan::token_params(0, 33));
            graph.run(gpu);
            compare(second, x, 33, bits);
        }
        {  // dequantize_matches_cpu
            const size_t tokens = 9;
            QuantRows cache(gpu, bits, VALUES, 64);
            std::vector<float> x(tokens * VALUES);
            orc_quant_rows(x.data(), tokens, VALUES);
            View xb(gpu.buffer_from(x)), out(gpu.buffer(tokens * VALUES * 2));
            cache.encode(gpu, xb, 0, tokens);
            cache.encode_dequantize(gpu, out, tokens);
            gpu.sync();
            const size_t groups = tokens * cache.per_token;
            auto data = gpu::contents<uint32_t>(cache.data, groups * kv_quant::words_per_group(bits));
            auto scales = gpu::contents<uint16_t>(cache.scales, groups);
            auto biases = gpu::contents<uint16_t>(cache.biases, groups);
            std::vector<float> want(tokens * VALUES);
            orc_dequantize(data.data(), scales.data(), biases.data(), groups, int(kv_quant::bits(bits)), want.data());
            auto got = gpu::contents<uint16_t>(out.buffer, tokens * VALUES);
            size_t bad = 0;
            for (size_t i = 0; i < got.size(); i++) bad += got[i] != orc_f32_to_f16(want[i]);
            EXPECT(bad == 0, "dequantize: %zu halves differ", bad);
        }
        {  // quantized_matches_cpu (tests/attention.rs:98-201)
            const size_t capacity = 1024;
            std::vector<float> q(HEADS * DIM), qg(HEADS * 2 * DIM), keys(capacity * KV * DIM), values(capacity * KV * DIM);
            orc_noise(q.data(), q.size(), 3);
            orc_noise(qg.data(), qg.size(), 4);
            orc_noise(keys.data(), keys.size(), 1);
            for (auto &k : keys) k *= 4.0f;
            orc_noise(values.data(), values.size(), 2);
            QuantRows kc(gpu, bits, VALUES, capacity), vc(gpu, bits, VALUES, capacity);
            View kx(gpu.buffer_from(keys)), vx(gpu.buffer_from(values));
            kc.encode(gpu, kx, 0, capacity);
            vc.encode(gpu, vx, 0, capacity);
            gpu.sync();
            const size_t groups = capacity * 8, words = kv_quant::words_per_group(bits);
            std::vector<float> kf(keys.size()), vf(values.size());
            {
                auto d = gpu::contents<uint32_t>(kc.data, groups * words);
                auto s = gpu::contents<uint16_t>(kc.scales, groups);
                auto z = gpu::contents<uint16_t>(kc.biases, groups);
                orc_dequantize(d.data(), s.data(), z.data(), groups, int(kv_quant::bits(bits)), kf.data());
                d = gpu::contents<uint32_t>(vc.data, groups * words);
                s = gpu::contents<uint16_t>(vc.scales, groups);
                z = gpu::contents<uint16_t>(vc.biases, groups);
                orc_dequantize(d.data(), s.data(), z.data(), groups, int(kv_quant::bits(bits)), vf.data());
            }
            View qb(gpu.buffer_from(q)), gb(gpu.buffer_from(qg)), out(gpu.buffer(HEADS * DIM * 4));
            attention::DecodeAttention att(gpu, HEADS, KV, DIM, capacity);
            plan::Plan plan(gpu);
            att.record_quant(plan, qb, kc, vc, gb, out);
            auto built = plan.build();
            auto replay = plan.build(true);  // the same launches as one HIP graph
            EXPECT(replay.is_graph(), "plan was not captured");
            for (size_t len : {1, 127, 129, 1000, 1024}) {
                plan.set_params(plan::token_params(0, uint32_t(len - 1)));
                // serial == replay, exactly (tests/plan.rs:27-45)
                replay.run(gpu);
                const auto from_graph = gpu::contents<float>(out.buffer, HEADS * DIM);
                hip_check(hipMemset(out.buffer.get(), 0xff, HEADS * DIM * 4), "hipMemset");
                built.run(gpu);
                EXPECT(std::memcmp(from_graph.data(), gpu::contents<float>(out.buffer, HEADS * DIM).data(), HEADS * DIM * 4) == 0,
                       "%d-bit len %zu: graph replay differs from the serial run", int(kv_quant::bits(bits)), len);
                auto got = gpu::contents<float>(out.buffer, HEADS * DIM);
                std::vector<double> want(HEADS * DIM);
                orc_attention_f64(q.data(), kf.data(), vf.data(), qg.data(), len, HEADS, KV, DIM, want.data(), 4);
                double worst = 0;
                for (size_t i = 0; i < got.size(); i++) worst = std::fmax(worst, std::fabs(double(got[i]) - want[i]));
                std::printf("%d-bit len %zu: worst error %.2e\n", int(kv_quant::bits(bits)), len, worst);
                EXPECT(worst < 2e-5, "%d-bit len %zu: %g", int(kv_quant::bits(bits)), len, worst);
            }
        }
    }
    // The module functions of src/kv_quant.rs (quantize, dequantize, round_trip, round_trip_as_half,
    // test_slack) and attention_prefill::spread, against the oracle.
    for (KvBits bits : {KvBits::Eight, KvBits::Four}) {
        const int b = int(kv_quant::bits(bits));
        std::vector<float> x(9 * VALUES);
        orc_quant_rows(x.data(), 9, VALUES);
        const size_t groups = x.size() / 64, words = kv_quant::words_per_group(bits);
        std::vector<uint32_t> wd(groups * words);
        std::vector<uint16_t> ws(groups), wz(groups);
        orc_quantize(x.data(), x.size(), b, wd.data(), ws.data(), wz.data());
        const auto q = kv_quant::quantize(gpu, x, bits);
        EXPECT(q.data == wd && q.scales == ws && q.biases == wz, "%d-bit quantize() differs from the CPU", b);
        std::vector<float> want(x.size());
        orc_dequantize(wd.data(), ws.data(), wz.data(), groups, b, want.data());
        const auto back = kv_quant::round_trip(gpu, x, bits);
        EXPECT(std::memcmp(back.data(), want.data(), want.size() * 4) == 0, "%d-bit round_trip differs", b);
        const auto half = kv_quant::round_trip_as_half(gpu, x, bits);
        size_t off = 0;
        for (size_t i = 0; i < want.size(); i++) off += half[i] != orc_f32_to_f16(want[i]);
        EXPECT(off == 0, "%d-bit round_trip_as_half: %zu values differ", b, off);
        EXPECT(kv_quant::test_slack(bits) == (b == 8 ? 4.0f : 16.0f), "test_slack");
    }
    {
        const auto s = attention_prefill::spread(4000, 2);
        size_t off = 0;
        for (size_t i = 0; i < s.size(); i++) {
            off += s[i] != orc_f32_to_f16(float((i * 7919 + 2 * 104729) % 1999) / 500.0f - 2.0f);
        }
        EXPECT(off == 0 && s.size() == 4000, "spread: %zu values differ", off);
    }
    {   // record_store: the codes it writes are the quantizer's codes of the key it reports
        const size_t pos = 41, capacity = 64;
        std::vector<float> qg(HEADS * 2 * DIM), k(KV * DIM), v(KV * DIM), ones(DIM, 1.0f);
        orc_noise(qg.data(), qg.size(), 21);
        orc_noise(k.data(), k.size(), 22);
        orc_noise(v.data(), v.size(), 23);
        QuantRows kc(gpu, KvBits::Eight, VALUES, capacity), vc(gpu, KvBits::Eight, VALUES, capacity);
        View q(gpu.buffer(HEADS * DIM * 4)), kb(gpu.buffer(KV * DIM * 4));
        plan::Plan plan(gpu);
        gpu_layers::record_store(plan, View(gpu.buffer_from(qg)), View(gpu.buffer_from(k)), View(gpu.buffer_from(v)),
                                 View(gpu.buffer_from(ones)), View(gpu.buffer_from(ones)), q, kc, vc,
                                 gpu_layers::prep_params(HEADS, KV, DIM, 64, 1e7f, 1e-6f), capacity, 1, &kb);
        plan.set_params(plan::token_params(0, uint32_t(pos)));
        plan.build(true).run(gpu);
        compare(kc, gpu::contents<float>(kb.buffer, KV * DIM), pos, KvBits::Eight);
        compare(vc, v, pos, KvBits::Eight);
    }
    {   // GpuDeltaNet::record_rows "as m calls of record would" (src/gpu_layers.rs:686-688), the snapshots
        // and record_restore (src/gpu_layers.rs:838-856; the reference's test at :1063-1095 restores a row
        // and goes on from there)
        const size_t kh = 2, vh = 4, dv = 16, kernel = 4, m = 5, key = kh * 128, val = vh * dv, ch = 2 * key + val;
        const size_t conv_n = (kernel - 1) * ch, state_n = vh * dv * 128;
        std::vector<float> x(m * ch), z(m * val), a(m * vh), b(m * vh), w(ch * kernel), alog(vh), dtb(vh), norm(dv, 1.0f);
        orc_noise(x.data(), x.size(), 31), orc_noise(z.data(), z.size(), 32), orc_noise(a.data(), a.size(), 33);
        orc_noise(b.data(), b.size(), 34), orc_noise(w.data(), w.size(), 35), orc_noise(alog.data(), vh, 36);
        orc_noise(dtb.data(), vh, 37);
        View xd(gpu.buffer_from(x)), zd(gpu.buffer_from(z)), ad(gpu.buffer_from(a)), bd(gpu.buffer_from(b));
        View wd(gpu.buffer_from(w)), al(gpu.buffer_from(alog)), dt(gpu.buffer_from(dtb)), nw(gpu.buffer_from(norm));
        View conv1(gpu.buffer(conv_n * 4)), st1(gpu.buffer(state_n * 4)), mixed1(gpu.buffer(m * ch * 4)), y1(gpu.buffer(m * val * 4));
        View conv2(gpu.buffer(conv_n * 4)), st2(gpu.buffer(state_n * 4)), mixed2(gpu.buffer(m * ch * 4)), y2(gpu.buffer(m * val * 4));
        View csn(gpu.buffer(m * conv_n * 4)), ssn(gpu.buffer(m * state_n * 4));
        plan::Plan one(gpu), many(gpu);
        for (size_t t = 0; t < m; t++) {
            const View mt = mixed1.at(t * ch * 4);
            deltanet::conv(one, xd.at(t * ch * 4), wd, conv1, mt, ch, kernel);
            deltanet::step(one, mt, mt.at(key * 4), mt.at(2 * key * 4), ad.at(t * vh * 4), bd.at(t * vh * 4), al, dt, st1,
                           zd.at(t * val * 4), nw, y1.at(t * val * 4), kh, vh, dv, 1e-6f);
        }
        {   // deltanet::token == conv then step
            View conv3(gpu.buffer(conv_n * 4)), st3(gpu.buffer(state_n * 4)), y3(gpu.buffer(m * val * 4));
            plan::Plan fused(gpu);
            for (size_t t = 0; t < m; t++) {
                deltanet::token(fused, xd.at(t * ch * 4), wd, conv3, ad.at(t * vh * 4), bd.at(t * vh * 4), al, dt, st3,
                                zd.at(t * val * 4), nw, y3.at(t * val * 4), kh, vh, dv, kernel, 1e-6f);
            }
            one.build(false).run(gpu);
            fused.build(true).run(gpu);
            auto worst3 = [](const std::vector<float> &p, const std::vector<float> &q) {
                float d = 0;
                for (size_t i = 0; i < p.size(); i++) d = std::max(d, std::fabs(p[i] - q[i]));
                return d;
            };
            EXPECT(gpu::contents<float>(conv1.buffer, conv_n) == gpu::contents<float>(conv3.buffer, conv_n), "token: conv state");
            EXPECT(worst3(gpu::contents<float>(y1.buffer, m * val), gpu::contents<float>(y3.buffer, m * val)) < 2e-5f, "token: y");
            EXPECT(worst3(gpu::contents<float>(st1.buffer, state_n), gpu::contents<float>(st3.buffer, state_n)) < 2e-5f, "token: state");
            // `one` ran here: start its states again for the comparison below
            hip_check(hipMemset(conv1.ptr<void>(), 0, conv_n * 4), "memset");
            hip_check(hipMemset(st1.ptr<void>(), 0, state_n * 4), "memset");
        }
        deltanet::conv_rows(many, xd, wd, conv2, mixed2, ch, kernel, m, &csn);
        deltanet::rows(many, mixed2, ad, bd, al, dt, st2, zd, nw, y2, kh, vh, dv, m, 1e-6f, &ssn);
        one.build(false).run(gpu);
        many.build(true).run(gpu);
        auto worst = [](const std::vector<float> &p, const std::vector<float> &q) {
            float d = 0;
            for (size_t i = 0; i < p.size(); i++) d = std::max(d, std::fabs(p[i] - q[i]));
            return d;
        };
        EXPECT(gpu::contents<float>(mixed1.buffer, m * ch) == gpu::contents<float>(mixed2.buffer, m * ch), "conv_rows != m convs");
        EXPECT(gpu::contents<float>(conv1.buffer, conv_n) == gpu::contents<float>(conv2.buffer, conv_n), "conv state");
        EXPECT(worst(gpu::contents<float>(y1.buffer, m * val), gpu::contents<float>(y2.buffer, m * val)) < 2e-5f, "rows y");
        EXPECT(worst(gpu::contents<float>(st1.buffer, state_n), gpu::contents<float>(st2.buffer, state_n)) < 2e-5f, "rows state");
        EXPECT(gpu::contents<float>(ssn.buffer, state_n, (m - 1) * state_n * 4) == gpu::contents<float>(st2.buffer, state_n),
               "last snapshot is the state");
        if (m <= 8) {   // deltanet::rows_fused == conv_rows + rows, snapshots included
            View conv4(gpu.buffer(conv_n * 4)), st4(gpu.buffer(state_n * 4)), y4(gpu.buffer(m * val * 4));
            View csn4(gpu.buffer(m * conv_n * 4)), ssn4(gpu.buffer(m * state_n * 4));
            plan::Plan both(gpu);
            deltanet::rows_fused(both, xd, wd, conv4, ad, bd, al, dt, st4, zd, nw, y4, kh, vh, dv, kernel, m, 1e-6f, &csn4, &ssn4);
            both.build(true).run(gpu);
            EXPECT(gpu::contents<float>(conv2.buffer, conv_n) == gpu::contents<float>(conv4.buffer, conv_n), "rows_fused: conv state");
            EXPECT(gpu::contents<float>(csn.buffer, m * conv_n) == gpu::contents<float>(csn4.buffer, m * conv_n), "rows_fused: conv snapshots");
            EXPECT(worst(gpu::contents<float>(y2.buffer, m * val), gpu::contents<float>(y4.buffer, m * val)) < 2e-5f, "rows_fused: y");
            EXPECT(worst(gpu::contents<float>(ssn.buffer, m * state_n), gpu::contents<float>(ssn4.buffer, m * state_n)) < 2e-5f,
                   "rows_fused: state snapshots");
            EXPECT(gpu::contents<float>(ssn4.buffer, state_n, (m - 1) * state_n * 4) == gpu::contents<float>(st4.buffer, state_n),
                   "rows_fused: last snapshot is the state");
        }
        // accept two rows: restore the state after row 1, then rows 2.. again give the same end state
        plan::Plan again(gpu);
        deltanet::restore(again, csn, ssn, 1, conv2, st2, conv_n, state_n);
        deltanet::conv_rows(again, xd.at(2 * ch * 4), wd, conv2, mixed2, ch, kernel, m - 2);
        deltanet::rows(again, mixed2, ad.at(2 * vh * 4), bd.at(2 * vh * 4), al, dt, st2, zd.at(2 * val * 4), nw, y2, kh, vh, dv,
                       m - 2, 1e-6f);
        again.build(false).run(gpu);
        EXPECT(gpu::contents<float>(ssn.buffer, state_n, (m - 1) * state_n * 4) == gpu::contents<float>(st2.buffer, state_n),
               "restore + the remaining rows");
        EXPECT(gpu::contents<float>(conv1.buffer, conv_n) == gpu::contents<float>(conv2.buffer, conv_n), "restore conv");
    }
    {   // GpuKvCache::resize keeps the rows (src/gpu_layers.rs:255-293); RowBackup puts rows back (src/gpu_cache.rs:196-283)
        gpu_layers::GpuKvCache cache(gpu, HEADS, KV, DIM, 200, KvBits::Eight);
        EXPECT(cache.capacity == 256 && cache.buffers().size() == 6, "GpuKvCache::with_bits");
        std::vector<float> x(150 * VALUES);
        orc_quant_rows(x.data(), 150, VALUES);
        const View xd(gpu.buffer_from(x));
        cache.quant->first.encode(gpu, xd, 0, 150);
        cache.quant->second.encode(gpu, xd, 0, 150);
        gpu.sync();
        const auto codes = gpu::contents<uint32_t>(cache.keys, 150 * 8 * 16);
        const auto scales = gpu::contents<uint16_t>(cache.quant->second.scales, 150 * 8);
        cache.resize(gpu, 1000);
        EXPECT(cache.capacity == 1024 && cache.keys.length() == 1024 * 8 * 16 * 4, "resize capacity");
        EXPECT(gpu::contents<uint32_t>(cache.keys, 150 * 8 * 16) == codes, "resize moved the codes");
        EXPECT(gpu::contents<uint16_t>(cache.quant->second.scales, 150 * 8) == scales, "resize moved the scales");
        EXPECT(cache.quant->first.data.get() == cache.keys.get(), "QuantRows follows the cache");
        compare(cache.quant->first, x, 0, KvBits::Eight);
        gpu_layers::RowBackup backup;
        backup.save(gpu, {&cache}, 100, 12);
        EXPECT(backup.bytes() == 12 * 1088, "RowBackup::bytes %zu", backup.bytes());
        std::vector<float> other(12 * VALUES, 0.25f);
        const View od(gpu.buffer_from(other));
        cache.quant->first.encode(gpu, od, 100, 12);
        cache.quant->second.encode(gpu, od, 100, 12);
        gpu.sync();
        EXPECT(gpu::contents<uint32_t>(cache.keys, 150 * 8 * 16) != codes, "the detour wrote over the rows");
        backup.restore(gpu, {&cache});
        EXPECT(backup.bytes() == 0 && gpu::contents<uint32_t>(cache.keys, 150 * 8 * 16) == codes, "RowBackup::restore");
        EXPECT(gpu::contents<uint16_t>(cache.quant->second.scales, 150 * 8) == scales, "RowBackup::restore scales");
        cache.resize(gpu, 100);
        EXPECT(cache.capacity == 128, "shrink");
        std::vector<float> first(x.begin(), x.begin() + 128 * VALUES);
        compare(cache.quant->first, first, 0, KvBits::Eight);
    }
    {   // a prefill chunk over a half cache of spread data (tests/attention_prefill.rs:14-60, shape (1000, 64)) by
        // the flash kernel and by AttGemm in two slices, against the CPU token by token
        const size_t pos = 1000, tokens = 64, n = pos + tokens, capacity = 1088;
        const auto qh = attention_prefill::spread(tokens * HEADS * DIM, 1);
        const auto kh = attention_prefill::spread(capacity * VALUES, 2), vh = attention_prefill::spread(capacity * VALUES, 3);
        std::vector<float> gate(tokens * HEADS * 2 * DIM);
        for (size_t i = 0; i < gate.size(); i++) gate[i] = float(i % 7) - 3.0f;
        auto widen = [](const std::vector<uint16_t> &h, size_t count) {
            std::vector<float> f(count);
            for (size_t i = 0; i < count; i++) {
                _Float16 x;
                std::memcpy(&x, &h[i], 2);
                f[i] = float(x);
            }
            return f;
        };
        std::vector<float> want(tokens * HEADS * DIM);
        const auto qf = widen(qh, qh.size()), kf = widen(kh, n * VALUES), vf = widen(vh, n * VALUES);
        orc_prefill(qf.data(), kf.data(), vf.data(), pos, tokens, HEADS, KV, DIM, gate.data(), want.data(), 8);
        View q(gpu.buffer_from(qh)), k(gpu.buffer_from(kh)), v(gpu.buffer_from(vh)), g(gpu.buffer_from(gate));
        View flash(gpu.buffer(want.size() * 4)), gemm(gpu.buffer(want.size() * 4));
        const attention_prefill::FlashParams f{uint32_t(HEADS), uint32_t(KV), uint32_t(pos), uint32_t(tokens), 1.0f / 16.0f};
        attention_prefill::encode(gpu, attention_prefill::DEFAULT, q, k, v, g, flash, f);
        setenv("SAETTA_AG_SLICES", "2", 1);
        const attention_gemm::AttGemm att(gpu, tokens, KV);
        unsetenv("SAETTA_AG_SLICES");
        EXPECT(att.slice == 32 && att.rows_pad == 256 && attention_gemm::KEYS == 1024, "AttGemm::new: slice %zu", att.slice);
        att.encode(gpu, q, k, v, nullptr, g, gemm, f);
        gpu.sync();
        const auto a = gpu::contents<float>(flash.buffer, want.size()), b = gpu::contents<float>(gemm.buffer, want.size());
        float worst_a = 0.0f, worst_b = 0.0f;
        for (size_t i = 0; i < want.size(); i++) {
            worst_a = std::max(worst_a, std::fabs(a[i] - want[i]));
            worst_b = std::max(worst_b, std::fabs(b[i] - want[i]));
        }
        std::printf("prefill (1000, 64): flash worst %.2e, gemm worst %.2e\n", worst_a, worst_b);
        EXPECT(worst_a < 2e-3f && worst_b < 2e-3f, "prefill chunk: flash %g gemm %g", worst_a, worst_b);
    }
    // shape checks panic (throw) as the reference asserts
    bool threw = false;
    try {
        attention::DecodeAttention bad(gpu, 16, 2, 128, 1024);
    } catch (const std::runtime_error &) {
        threw = true;
    }
    EXPECT(threw, "DecodeAttention accepted head dim 128");
    std::printf(failures ? "%d FAILURES\n" : "all host tests passed\n", failures);
    return failures ? 1 : 0;
}
