// Host side of the attention hot path in C++, above the C ABI of include/saetta_hip.h.
//
// The reference's host code for this path is Rust calling Metal; this header mirrors its public
// items one for one (same names, argument meaning, ownership and error behaviour) so that a
// caller of src/kv_quant.rs, src/attention.rs, src/rows.rs and src/attention_prefill.rs finds
// the same surface:
//
//   gpu::Gpu, gpu::Buffer, View        src/gpu.rs:233-290, src/qmv.rs:18-23
//   plan::TokenParams, Plan, Built     src/plan.rs:16-35, 63-146, 187-273
//   kv_quant::KvBits, GROUP, QuantRows src/kv_quant.rs:8-50, 156-283
//   attention::DecodeAttention         src/attention.rs:28-171
//   rows::MAX_ROWS, AttentionRows      src/rows.rs:8-9, 344-494
//   attention_prefill::FlashParams, KERNELS, DEFAULT, KEY_BLOCK, encode
//                                      src/attention_prefill.rs:4-72
//   attention_gemm::KEYS, AttGemm      src/attention_gemm.rs:28, 95-364
//
// Where the reference asserts or panics, these throw std::runtime_error.  Buffers are
// reference-counted and zero-filled like Metal's (src/gpu.rs:287-290); a Plan keeps every
// buffer it binds alive (src/plan.rs:113-123).  Single-threaded use, like the reference's Gpu.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/saetta_hip.h"

namespace saetta {

inline void check(int rc, const char *what) {
    if (rc != 0) throw std::runtime_error(std::string(what) + ": " + saetta_last_error() + " (code " + std::to_string(rc) + ")");
}
inline void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
// The current device's sticky status word: 0 unless a kernel's bounded wait gave up, after which every call on the
// device fails (check() throws) until the word is cleared.  The reference asserts on its command buffers' status.
inline uint32_t device_status(bool clear = false) { return saetta_device_status(clear ? 1 : 0); }

namespace gpu {

// A device allocation, zero-filled, freed when the last handle goes.
class Buffer {
  public:
    Buffer() = default;
    explicit Buffer(size_t bytes) : bytes_(bytes) {
        void *p = nullptr;
        hip_check(hipMalloc(&p, bytes ? bytes : 1), "hipMalloc");
        hip_check(hipMemset(p, 0, bytes ? bytes : 1), "hipMemset");
        ptr_ = std::shared_ptr<void>(p, [](void *q) { (void)hipFree(q); });
    }
    void *get() const { return ptr_.get(); }
    size_t length() const { return bytes_; }

  private:
    std::shared_ptr<void> ptr_;
    size_t bytes_ = 0;
};

// Device + stream (Gpu::new, src/gpu.rs:233-263).
class Gpu {
  public:
    Gpu() {
        check(saetta_init(), "Gpu::new");
        hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
    }
    ~Gpu() { (void)hipStreamDestroy(stream_); }
    Gpu(const Gpu &) = delete;
    Gpu &operator=(const Gpu &) = delete;
    Buffer buffer(size_t bytes) const { return Buffer(bytes); }
    template <typename T>
    Buffer buffer_from(const std::vector<T> &data) const {
        Buffer b(data.size() * sizeof(T));
        hip_check(hipMemcpy(b.get(), data.data(), data.size() * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy");
        return b;
    }
    hipStream_t stream() const { return stream_; }
    void sync() const { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }

  private:
    hipStream_t stream_ = nullptr;
};

// contents::<T>(buffer, n) of src/gpu.rs: a host copy of the first n elements.
template <typename T>
std::vector<T> contents(const Buffer &b, size_t n, size_t byte_offset = 0) {
    std::vector<T> out(n);
    hip_check(hipMemcpy(out.data(), static_cast<char *>(b.get()) + byte_offset, n * sizeof(T), hipMemcpyDeviceToHost),
              "hipMemcpy");
    return out;
}

}  // namespace gpu

// A buffer and a byte offset into it (src/qmv.rs:18-23).
struct View {
    gpu::Buffer buffer;
    uint64_t offset = 0;
    View() = default;
    explicit View(gpu::Buffer b, uint64_t off = 0) : buffer(std::move(b)), offset(off) {}
    template <typename T>
    T *ptr() const { return reinterpret_cast<T *>(static_cast<char *>(buffer.get()) + offset); }
    View at(uint64_t bytes) const { return View(buffer, offset + bytes); }
};

namespace plan {

using TokenParams = saetta_token_params;
inline TokenParams token_params(uint32_t token, uint32_t position) {  // TokenParams::new
    return TokenParams{token, position, position + 1, 0};
}

class Built {
  public:
    using Ops = std::vector<std::pair<std::string, std::function<void(hipStream_t)>>>;
    // graph: the launches are captured once into a HIP graph (the counterpart of the reference's
    // indirect command buffer, src/plan.rs:229-235) and every run is one graph launch.  Every
    // entry point of the library only enqueues kernels, so a plan can always be captured, with
    // one exception: prefill without a caller's workspace allocates.
    Built(Ops ops, const gpu::Gpu &gpu, bool graph) : ops_(std::move(ops)) {
        if (!graph || ops_.empty()) return;
        // The library's one-time set-up must not happen under capture; the launches themselves are not
        // run here: a plan may hold ops that advance a state (the DeltaNet ones do).
        if (int rc = saetta_init()) throw std::runtime_error(std::string("saetta_init: ") + saetta_last_error() + " (" + std::to_string(rc) + ")");
        gpu.sync();
        hipGraph_t g = nullptr;
        hip_check(hipStreamBeginCapture(gpu.stream(), hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
        try {
            for (auto &op : ops_) op.second(gpu.stream());
        } catch (...) {
            // an op that refuses its arguments must not leave the stream capturing
            (void)hipStreamEndCapture(gpu.stream(), &g);
            if (g) (void)hipGraphDestroy(g);
            throw;
        }
        hip_check(hipStreamEndCapture(gpu.stream(), &g), "hipStreamEndCapture");
        hipGraphExec_t e = nullptr;
        hip_check(hipGraphInstantiate(&e, g, nullptr, nullptr, 0), "hipGraphInstantiate");
        hip_check(hipGraphDestroy(g), "hipGraphDestroy");
        exec_ = std::shared_ptr<hipGraphExec>(e, [](hipGraphExec_t x) { (void)hipGraphExecDestroy(x); });
    }
    // Replays the recorded launches and waits (Built::run, src/plan.rs:241-243); the wall time in seconds.
    double run(const gpu::Gpu &gpu) const { return run_timed(gpu).first; }
    // `run`, also returning the GPU's own time between the first launch and the end of the last,
    // in seconds (Built::run_timed, src/plan.rs:249-251), from two events on the stream.
    std::pair<double, double> run_timed(const gpu::Gpu &gpu) const {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        hip_check(hipEventCreate(&e0), "hipEventCreate");
        hip_check(hipEventCreate(&e1), "hipEventCreate");
        const auto start = std::chrono::steady_clock::now();
        hip_check(hipEventRecord(e0, gpu.stream()), "hipEventRecord");
        enqueue(gpu);
        hip_check(hipEventRecord(e1, gpu.stream()), "hipEventRecord");
        hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
        const double wall = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
        float ms = 0.0f;
        hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        return {wall, double(ms) * 1e-3};
    }
    // `run` without the wait (Built::commit, src/plan.rs:254-256): what is returned waits for it.
    struct Pending {
        std::shared_ptr<ihipEvent_t> done;
        void wait() const { hip_check(hipEventSynchronize(done.get()), "hipEventSynchronize"); }
    };
    Pending commit(const gpu::Gpu &gpu) const {
        hipEvent_t e = nullptr;
        hip_check(hipEventCreate(&e), "hipEventCreate");
        enqueue(gpu);
        hip_check(hipEventRecord(e, gpu.stream()), "hipEventRecord");
        return Pending{std::shared_ptr<ihipEvent_t>(e, [](hipEvent_t x) { (void)hipEventDestroy(x); })};
    }
    // Replays without waiting and without an event, for timing many runs back to back.
    void enqueue(const gpu::Gpu &gpu) const {
        if (exec_) {
            hip_check(hipGraphLaunch(exec_.get(), gpu.stream()), "hipGraphLaunch");
        } else {
            for (auto &op : ops_) op.second(gpu.stream());
        }
    }
    bool is_graph() const { return bool(exec_); }

  private:
    Ops ops_;
    std::shared_ptr<hipGraphExec> exec_;
};

// A list of launches recorded once and run for every token; what changes per token is in the
// TokenParams buffer, which the kernels read when they run.
class Plan {
  public:
    explicit Plan(const gpu::Gpu &gpu) : params(gpu.buffer(sizeof(TokenParams))), gpu_(gpu) {
        // set_params copies from pinned memory, so that the copy is ordered by the stream and needs no wait:
        // a ring of slots, each guarded by the event of the copy that last read it
        TokenParams *ring = nullptr;
        hip_check(hipHostMalloc(reinterpret_cast<void **>(&ring), RING * sizeof(TokenParams), hipHostMallocDefault), "hipHostMalloc");
        ring_ = std::shared_ptr<TokenParams>(ring, [](TokenParams *x) { (void)hipHostFree(x); });
        for (int i = 0; i < RING; i++) {
            hipEvent_t e = nullptr;
            hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
            read_[i] = std::shared_ptr<ihipEvent_t>(e, [](hipEvent_t x) { (void)hipEventDestroy(x); });
        }
    }
    View params;
    void op(std::string kernel, std::function<void(hipStream_t)> launch) { ops_.emplace_back(std::move(kernel), std::move(launch)); }
    // Plan::set_params (src/plan.rs:144-146): a small copy on the stream, in order with the runs around it.
    void set_params(TokenParams tp) {
        const int slot = next_;
        next_ = (next_ + 1) % RING;
        if (used_[slot]) hip_check(hipEventSynchronize(read_[slot].get()), "hipEventSynchronize");  // (RING copies ago: long done)
        ring_.get()[slot] = tp;
        hip_check(hipMemcpyAsync(params.ptr<void>(), ring_.get() + slot, sizeof tp, hipMemcpyHostToDevice, gpu_.stream()), "set_params");
        hip_check(hipEventRecord(read_[slot].get(), gpu_.stream()), "hipEventRecord");
        used_[slot] = true;
    }
    const gpu::Gpu &gpu() const { return gpu_; }
    size_t len() const { return ops_.size(); }
    bool is_empty() const { return ops_.empty(); }
    // A buffer holding `data`, for values that never change between tokens (Plan::constant, src/plan.rs:128-141).
    template <typename T>
    View constant(const std::vector<T> &data) const {
        return View(gpu_.buffer_from(data));
    }
    // Launches every op one after the other on the stream, outside any graph, and waits
    // (Plan::run_serial, src/plan.rs:157-168); the wall time in seconds.
    double run_serial() const {
        const auto start = std::chrono::steady_clock::now();
        for (auto &op : ops_) op.second(gpu_.stream());
        gpu_.sync();
        return std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    }
    // Each kernel name with how many ops use it, in order of first use (Plan::kernels, src/plan.rs:171-181).
    std::vector<std::pair<std::string, size_t>> kernels() const {
        std::vector<std::pair<std::string, size_t>> out;
        for (auto &op : ops_) {
            auto it = std::find_if(out.begin(), out.end(), [&](const auto &k) { return k.first == op.first; });
            if (it == out.end()) {
                out.emplace_back(op.first, 1);
            } else {
                it->second++;
            }
        }
        return out;
    }
    Built build(bool graph = false) const { return Built(ops_, gpu_, graph); }
    // Only the launches whose kernel name `keep` accepts (Plan::build_where, src/plan.rs:237-273).
    Built build_where(const std::function<bool(const std::string &)> &keep, bool graph = false) const {
        Built::Ops kept;
        for (auto &op : ops_) {
            if (keep(op.first)) kept.push_back(op);
        }
        return Built(std::move(kept), gpu_, graph);
    }

  private:
    std::vector<std::pair<std::string, std::function<void(hipStream_t)>>> ops_;
    const gpu::Gpu &gpu_;
    static constexpr int RING = 8;
    std::shared_ptr<TokenParams> ring_;
    std::shared_ptr<ihipEvent_t> read_[RING];
    bool used_[RING] = {};
    int next_ = 0;
};

}  // namespace plan

namespace kv_quant {

constexpr size_t GROUP = 64;

enum class KvBits { Half, Eight, Four };

inline bool parse(const std::string &s, KvBits &out) {
    if (s == "16") return out = KvBits::Half, true;
    if (s == "8") return out = KvBits::Eight, true;
    if (s == "4") return out = KvBits::Four, true;
    return false;
}
inline uint32_t bits(KvBits b) { return b == KvBits::Half ? 16 : b == KvBits::Eight ? 8 : 4; }
inline size_t words_per_group(KvBits b) { return 2 * bits(b); }
inline double bytes_per_value(KvBits b) { return b == KvBits::Half ? 2.0 : bits(b) / 8.0 + 4.0 / GROUP; }

// The codes, scales and biases of one cache (keys or values).
struct QuantRows {
    gpu::Buffer data, scales, biases;
    KvBits bits;
    size_t per_token;

    QuantRows(const gpu::Gpu &gpu, KvBits b, size_t values, size_t capacity) : bits(b), per_token(values / GROUP) {
        if (b == KvBits::Half || values % GROUP != 0) throw std::runtime_error("QuantRows::new: bits must be 8 or 4, values a multiple of 64");
        const size_t groups = per_token * capacity;
        data = gpu.buffer(groups * words_per_group(b) * 4);
        scales = gpu.buffer(groups * 2);
        biases = gpu.buffer(groups * 2);
    }
    saetta_quant_rows c() const {
        return saetta_quant_rows{static_cast<uint32_t *>(data.get()), static_cast<uint16_t *>(scales.get()),
                                 static_cast<uint16_t *>(biases.get())};
    }
    // One token's values x into its slot, at the plan's position.
    void record(plan::Plan &plan, const View &x) const { record_at(plan, x, plan.params, false); }
    void record_at(plan::Plan &plan, const View &x, const View &params, bool /*parallel*/) const {
        const saetta_kv_quant_params p{uint32_t(per_token), uint32_t(per_token)};
        const QuantRows self = *this;
        const int nbits = int(kv_quant::bits(bits));
        plan.op(nbits == 8 ? "kv_quantize_8" : "kv_quantize_4", [=](hipStream_t s) {
            check(saetta_kv_quantize(s, nbits, x.ptr<float>(), self.c(), p, params.ptr<saetta_token_params>(), 0), "kv_quantize");
        });
    }
    // `tokens` tokens of x into the slots from pos.
    void encode(const gpu::Gpu &gpu, const View &x, size_t pos, size_t tokens) const {
        const saetta_kv_quant_params p{uint32_t(per_token * tokens), uint32_t(per_token)};
        check(saetta_kv_quantize(gpu.stream(), int(kv_quant::bits(bits)), x.ptr<float>(), c(), p, nullptr, uint32_t(pos)), "kv_quantize");
    }
    // Tokens 0..tokens as half into out.
    void encode_dequantize(const gpu::Gpu &gpu, const View &out, size_t tokens) const {
        const saetta_kv_quant_params p{uint32_t(per_token * tokens), uint32_t(per_token)};
        check(saetta_kv_dequantize(gpu.stream(), int(kv_quant::bits(bits)), c(), out.ptr<uint16_t>(), p), "kv_dequantize");
    }
};

// The CPU-side functions of src/kv_quant.rs:54-135 with host vectors in and out; the arithmetic
// runs on the device (the same kernels the cache uses), so the results are the cache's own.
struct Quantized {
    std::vector<uint32_t> data;
    std::vector<uint16_t> scales, biases;  // f16 bits
};

template <typename T>
inline std::vector<T> download(const gpu::Gpu &gpu, const gpu::Buffer &b, size_t n) {
    gpu.sync();
    return gpu::contents<T>(b, n);
}

inline Quantized quantize(const gpu::Gpu &gpu, const std::vector<float> &x, KvBits b) {
    if (x.size() % GROUP != 0) throw std::runtime_error("quantize: length must be a multiple of 64");
    const size_t groups = x.size() / GROUP;
    QuantRows rows(gpu, b, GROUP, groups);
    rows.encode(gpu, View(gpu.buffer_from(x)), 0, groups);
    return Quantized{download<uint32_t>(gpu, rows.data, groups * words_per_group(b)), download<uint16_t>(gpu, rows.scales, groups),
                     download<uint16_t>(gpu, rows.biases, groups)};
}

inline std::vector<float> dequantize(const gpu::Gpu &gpu, const Quantized &q, KvBits b) {
    const size_t groups = q.scales.size();
    if (b == KvBits::Half || q.data.size() != groups * words_per_group(b) || q.biases.size() != groups)
        throw std::runtime_error("dequantize: sizes do not match the bit width");
    const gpu::Buffer data = gpu.buffer_from(q.data), scales = gpu.buffer_from(q.scales), biases = gpu.buffer_from(q.biases);
    const gpu::Buffer out = gpu.buffer(groups * GROUP * 4);
    const saetta_quant_rows rows{static_cast<uint32_t *>(data.get()), static_cast<uint16_t *>(scales.get()),
                                 static_cast<uint16_t *>(biases.get())};
    check(saetta_kv_dequantize_f32(gpu.stream(), int(bits(b)), rows, static_cast<float *>(out.get()),
                                   saetta_kv_quant_params{uint32_t(groups), uint32_t(groups)}),
          "kv_dequantize_f32");
    return download<float>(gpu, out, groups * GROUP);
}

// x after a round trip through the cache, as a decode cache holds it.  (A half cache rounds to
// half; that case is left to the caller's own half type.)
inline std::vector<float> round_trip(const gpu::Gpu &gpu, const std::vector<float> &x, KvBits b) {
    if (b == KvBits::Half) throw std::runtime_error("round_trip: a half cache is a plain conversion to half");
    return dequantize(gpu, quantize(gpu, x, b), b);
}

// ... and through the half copy prefill attention reads (f16 bits).
inline std::vector<uint16_t> round_trip_as_half(const gpu::Gpu &gpu, const std::vector<float> &x, KvBits b) {
    const size_t groups = x.size() / GROUP;
    QuantRows rows(gpu, b, GROUP, groups);
    rows.encode(gpu, View(gpu.buffer_from(x)), 0, groups);
    const gpu::Buffer out = gpu.buffer(x.size() * 2);
    rows.encode_dequantize(gpu, View(out), groups);
    return download<uint16_t>(gpu, out, x.size());
}

inline float test_slack(KvBits b) { return b == KvBits::Half ? 1.0f : b == KvBits::Eight ? 4.0f : 16.0f; }

}  // namespace kv_quant

namespace gpu_layers {

using PrepParams = saetta_prep_params;
inline PrepParams prep_params(size_t heads, size_t kv_heads, size_t dim, size_t rope_dims, float rope_theta, float eps) {
    return PrepParams{uint32_t(heads), uint32_t(kv_heads), uint32_t(dim), uint32_t(rope_dims / 2), std::log2(rope_theta), eps};
}

// GpuAttention::record_store (src/gpu_layers.rs:370-411): q norm and RoPE into q, k norm and RoPE,
// then the token's key and value into the cache slot at the plan's position, in one launch where the
// reference records attention_prep{,_float} and two kv_quantize dispatches.  Half cache:
inline void record_store(plan::Plan &plan, const View &q_and_gate, const View &k, const View &v, const View &q_norm,
                         const View &k_norm, const View &q, const View &keys, const View &values, PrepParams p,
                         size_t capacity, size_t rows = 1) {
    const View tp = plan.params;
    plan.op("attention_prep_store", [=](hipStream_t s) {
        check(saetta_attn_prep_store(s, 16, q_and_gate.ptr<float>(), k.ptr<float>(), v.ptr<float>(), q_norm.ptr<float>(),
                                     k_norm.ptr<float>(), q.ptr<float>(), keys.ptr<uint16_t>(), values.ptr<uint16_t>(),
                                     saetta_quant_rows{}, saetta_quant_rows{}, nullptr, p, uint32_t(rows), uint32_t(capacity),
                                     tp.ptr<saetta_token_params>()),
              "attn_prep_store");
    });
}
// ... and a quantized cache; k_back (optional) gets the normed, rotated key in f32.
inline void record_store(plan::Plan &plan, const View &q_and_gate, const View &k, const View &v, const View &q_norm,
                         const View &k_norm, const View &q, const kv_quant::QuantRows &keys, const kv_quant::QuantRows &values,
                         PrepParams p, size_t capacity, size_t rows = 1, const View *k_back = nullptr) {
    const View tp = plan.params;
    const kv_quant::QuantRows kq = keys, vq = values;
    const int nbits = int(kv_quant::bits(keys.bits));
    const View kb = k_back ? *k_back : View();
    const bool has_kb = k_back != nullptr;
    plan.op("attention_prep_store", [=](hipStream_t s) {
        check(saetta_attn_prep_store(s, nbits, q_and_gate.ptr<float>(), k.ptr<float>(), v.ptr<float>(), q_norm.ptr<float>(),
                                     k_norm.ptr<float>(), q.ptr<float>(), nullptr, nullptr, kq.c(), vq.c(),
                                     has_kb ? kb.ptr<float>() : nullptr, p, uint32_t(rows), uint32_t(capacity),
                                     tp.ptr<saetta_token_params>()),
              "attn_prep_store");
    });
}

}  // namespace gpu_layers

namespace deltanet {

// Records deltanet_conv (kernels/layers.metal:203-226): depthwise causal conv1d + SiLU of one token;
// `state` [kernel_size - 1][channels] takes x in.
inline void conv(plan::Plan &plan, const View &x, const View &w, const View &state, const View &out, size_t channels,
                 size_t kernel_size) {
    const saetta_conv_params p{uint32_t(channels), uint32_t(kernel_size)};
    plan.op("deltanet_conv", [=](hipStream_t s) {
        check(saetta_deltanet_conv(s, x.ptr<float>(), w.ptr<float>(), state.ptr<float>(), out.ptr<float>(), p), "deltanet_conv");
    });
}

// Records deltanet_step (kernels/layers.metal:297-357): normalize_qk, the gates, the delta rule and
// the gated RMSNorm for every value head; key dim 128.
inline void step(plan::Plan &plan, const View &q, const View &k, const View &v, const View &a, const View &b, const View &a_log,
                 const View &dt_bias, const View &state, const View &z, const View &norm_w, const View &y, size_t k_heads,
                 size_t v_heads, size_t v_dim, float eps) {
    const saetta_step_params p{uint32_t(k_heads), uint32_t(v_heads), uint32_t(v_dim), eps};
    plan.op("deltanet_step", [=](hipStream_t s) {
        check(saetta_deltanet_step(s, q.ptr<float>(), k.ptr<float>(), v.ptr<float>(), a.ptr<float>(), b.ptr<float>(),
                                   a_log.ptr<float>(), dt_bias.ptr<float>(), state.ptr<float>(), z.ptr<float>(),
                                   norm_w.ptr<float>(), y.ptr<float>(), p),
              "deltanet_step");
    });
}

// One token, conv and step as one call of two launches with the state rows spread over more
// workgroups: what conv + step give, without the conv output in between (GpuDeltaNet::record,
// src/gpu_layers.rs:633-684).
inline void token(plan::Plan &plan, const View &x, const View &w, const View &conv_state, const View &a, const View &b,
                  const View &a_log, const View &dt_bias, const View &state, const View &z, const View &norm_w, const View &y,
                  size_t k_heads, size_t v_heads, size_t v_dim, size_t kernel_size, float eps) {
    const saetta_conv_params cp{uint32_t(2 * k_heads * 128 + v_heads * v_dim), uint32_t(kernel_size)};
    const saetta_step_params sp{uint32_t(k_heads), uint32_t(v_heads), uint32_t(v_dim), eps};
    plan.op("deltanet_token", [=](hipStream_t s) {
        check(saetta_deltanet_token(s, x.ptr<float>(), w.ptr<float>(), conv_state.ptr<float>(), a.ptr<float>(), b.ptr<float>(),
                                    a_log.ptr<float>(), dt_bias.ptr<float>(), state.ptr<float>(), z.ptr<float>(),
                                    norm_w.ptr<float>(), y.ptr<float>(), cp, sp),
              "deltanet_token");
    });
}

// Up to 8 rows, conv and step as one call of two launches (kernel deltanet_rows, GpuDeltaNet::record_rows
// with DN_SIMDS = 0, src/gpu_layers.rs:737-757): what conv_rows + rows give.  With the two snapshot
// buffers the conv and delta states after each row go there too.
inline void rows_fused(plan::Plan &plan, const View &x, const View &w, const View &conv_state, const View &a, const View &b,
                       const View &a_log, const View &dt_bias, const View &state, const View &z, const View &norm_w,
                       const View &y, size_t k_heads, size_t v_heads, size_t v_dim, size_t kernel_size, size_t rows, float eps,
                       const View *conv_snaps = nullptr, const View *state_snaps = nullptr) {
    if ((conv_snaps == nullptr) != (state_snaps == nullptr)) throw std::runtime_error("deltanet_rows_fused: both snapshot buffers or neither");
    const bool has = conv_snaps != nullptr;
    const saetta_rows_fused_params p{uint32_t(k_heads), uint32_t(v_heads), uint32_t(v_dim), uint32_t(kernel_size), eps,
                                     uint32_t(rows), has ? 1u : 0u};
    const View cs = has ? *conv_snaps : View{}, ss = has ? *state_snaps : View{};
    plan.op("deltanet_rows_fused", [=](hipStream_t s) {
        check(saetta_deltanet_rows_fused(s, x.ptr<float>(), w.ptr<float>(), conv_state.ptr<float>(), a.ptr<float>(),
                                         b.ptr<float>(), a_log.ptr<float>(), dt_bias.ptr<float>(), state.ptr<float>(),
                                         z.ptr<float>(), norm_w.ptr<float>(), y.ptr<float>(), has ? cs.ptr<float>() : nullptr,
                                         has ? ss.ptr<float>() : nullptr, p),
              "deltanet_rows_fused");
    });
}

// Records the conv of `tokens` tokens in order (conv_rows2 + conv_state, kernels/prefill.metal:734-786;
// deltanet_conv_rows, kernels/layers.metal:510-544).  x, out [tokens][channels]; with `snaps`
// ([tokens][kernel_size - 1][channels]) the state after each token goes there too.
inline void conv_rows(plan::Plan &plan, const View &x, const View &w, const View &state, const View &out, size_t channels,
                      size_t kernel_size, size_t tokens, const View *snaps = nullptr) {
    const saetta_conv_rows_params p{uint32_t(channels), uint32_t(kernel_size), uint32_t(tokens), snaps ? 1u : 0u};
    const View sn = snaps ? *snaps : View{};
    const bool has = snaps != nullptr;
    plan.op("deltanet_conv_rows", [=](hipStream_t s) {
        check(saetta_deltanet_conv_rows(s, x.ptr<float>(), w.ptr<float>(), state.ptr<float>(), out.ptr<float>(),
                                        has ? sn.ptr<float>() : nullptr, p),
              "deltanet_conv_rows");
    });
}

// Records the step of `tokens` tokens in order (delta_prep + delta_rows3 + the gated norm,
// kernels/prefill.metal:788-1116; deltanet_step_rows, GpuDeltaNet::record_rows, src/gpu_layers.rs:686-786).
// `mixed` [tokens][q | k | v] is the conv output; with `snaps` ([tokens][v_heads][v_dim][128]) the
// state after each token goes there too (GpuDeltaNetSnaps, src/gpu_layers.rs:819-836).
inline void rows(plan::Plan &plan, const View &mixed, const View &a, const View &b, const View &a_log, const View &dt_bias,
                 const View &state, const View &z, const View &norm_w, const View &y, size_t k_heads, size_t v_heads,
                 size_t v_dim, size_t tokens, float eps, const View *snaps = nullptr) {
    const saetta_rows_step_params p{uint32_t(k_heads), uint32_t(v_heads), uint32_t(v_dim), uint32_t(tokens), eps, snaps ? 1u : 0u};
    const View sn = snaps ? *snaps : View{};
    const bool has = snaps != nullptr;
    // a prefill chunk runs in blocks of 64 tokens and keeps per-block matrices in a workspace, which the
    // recorded op owns (the reference's prefill works in buffers of its own, src/prefill.rs:1433-1578)
    const size_t need = saetta_deltanet_rows_workspace_bytes(p);
    const gpu::Buffer ws = need ? gpu::Buffer(need) : gpu::Buffer();
    plan.op("deltanet_rows", [=](hipStream_t s) {
        check(saetta_deltanet_rows_ws(s, mixed.ptr<float>(), a.ptr<float>(), b.ptr<float>(), a_log.ptr<float>(),
                                      dt_bias.ptr<float>(), state.ptr<float>(), z.ptr<float>(), norm_w.ptr<float>(),
                                      y.ptr<float>(), has ? sn.ptr<float>() : nullptr, p, need ? ws.get() : nullptr, need),
              "deltanet_rows");
    });
}

// GpuDeltaNetSnaps::record_restore (src/gpu_layers.rs:838-856): the state after row `row` of the
// last rows call becomes the state; two device copies in stream order.
inline void restore(plan::Plan &plan, const View &conv_snaps, const View &state_snaps, size_t row, const View &conv,
                    const View &state, size_t conv_floats, size_t state_floats) {
    plan.op("copy_u32", [=](hipStream_t s) {
        hip_check(hipMemcpyAsync(conv.ptr<float>(), conv_snaps.ptr<float>() + row * conv_floats, conv_floats * 4,
                                 hipMemcpyDeviceToDevice, s), "restore conv");
        hip_check(hipMemcpyAsync(state.ptr<float>(), state_snaps.ptr<float>() + row * state_floats, state_floats * 4,
                                 hipMemcpyDeviceToDevice, s), "restore state");
    });
}

}  // namespace deltanet

namespace attention {

constexpr size_t DIM = 256;

class DecodeAttention {
  public:
    DecodeAttention(const gpu::Gpu &gpu, size_t heads, size_t kv_heads, size_t head_dim, size_t capacity)
        : heads_(heads), kv_heads_(kv_heads), capacity_(capacity) {
        if (head_dim != DIM) throw std::runtime_error("decode attention is written for head dim 256");
        if (heads != kv_heads * 8) throw std::runtime_error("decode attention needs 8 q heads per kv head");
        part_o_ = gpu.buffer(saetta_part_o_bytes(uint32_t(heads), uint32_t(capacity), 1));
        part_ml_ = gpu.buffer(saetta_part_ml_bytes(uint32_t(heads), uint32_t(capacity), 1));
    }
    // "attention_partial_mma": the library picks (the kernel with loader waves for one row over
    // codes in a large cache); "attention_partial": the register kernels only (src/attention.rs:36-38).
    std::string kernel = "attention_partial_mma";

    void record(plan::Plan &plan, const View &q, const View &keys, const View &values, const View &q_and_gate, const View &out) const {
        const auto p = params();
        const uint32_t flags = this->flags();
        const View tp = plan.params;
        const gpu::Buffer po = part_o_, pml = part_ml_;
        auto launch = [=](uint32_t stage) {
            return [=](hipStream_t s) {
                check(saetta_attn_decode(s, q.ptr<float>(), keys.ptr<uint16_t>(), values.ptr<uint16_t>(), static_cast<float *>(po.get()),
                                         static_cast<float *>(pml.get()), q_and_gate.ptr<float>(), out.ptr<float>(), p,
                                         tp.ptr<saetta_token_params>(), stage | flags),
                      "attn_decode");
            };
        };
        plan.op(kernel, launch(SAETTA_STAGE_PARTIAL));
        plan.op("attention_reduce", launch(SAETTA_STAGE_REDUCE));
    }
    void record_quant(plan::Plan &plan, const View &q, const kv_quant::QuantRows &keys, const kv_quant::QuantRows &values,
                      const View &q_and_gate, const View &out) const {
        if (keys.bits == kv_quant::KvBits::Half) throw std::runtime_error("a half cache goes through record");
        const auto p = params();
        const View tp = plan.params;
        const gpu::Buffer po = part_o_, pml = part_ml_;
        const kv_quant::QuantRows k = keys, v = values;
        const int nbits = int(kv_quant::bits(keys.bits));
        const uint32_t flags = this->flags();
        auto launch = [=](uint32_t stage) {
            return [=](hipStream_t s) {
                check(saetta_attn_decode_quant(s, nbits, q.ptr<float>(), k.c(), v.c(), static_cast<float *>(po.get()),
                                               static_cast<float *>(pml.get()), q_and_gate.ptr<float>(), out.ptr<float>(), p,
                                               tp.ptr<saetta_token_params>(), stage | flags),
                      "attn_decode_quant");
            };
        };
        plan.op(kernel + (nbits == 8 ? "_q8" : "_q4"), launch(SAETTA_STAGE_PARTIAL));
        plan.op("attention_reduce", launch(SAETTA_STAGE_REDUCE));
    }

  private:
    uint32_t flags() const {
        if (kernel == "attention_partial_mma") return 0;
        if (kernel == "attention_partial") return SAETTA_STAGE_NO_LOADERS;
        throw std::runtime_error("no decode attention kernel " + kernel);
    }
    saetta_decode_params params() const {
        return saetta_decode_params{uint32_t(heads_), uint32_t(kv_heads_), uint32_t(capacity_), 1.0f / std::sqrt(float(DIM))};
    }
    size_t heads_, kv_heads_, capacity_;
    gpu::Buffer part_o_, part_ml_;
};

}  // namespace attention

namespace rows {

constexpr size_t MAX_ROWS = 8;

class AttentionRows {
  public:
    AttentionRows(const gpu::Gpu &gpu, size_t heads, size_t kv_heads, size_t capacity, size_t rows)
        : heads_(heads), kv_heads_(kv_heads), capacity_(capacity), rows_(rows) {
        if (heads != kv_heads * 8) throw std::runtime_error("rows attention needs 8 q heads per kv head");
        if (rows < 1 || rows > MAX_ROWS) throw std::runtime_error(std::to_string(rows) + " rows");
        splits_ = saetta_part_ml_bytes(uint32_t(heads), uint32_t(capacity), 1) / (heads * 8);
        part_o_ = gpu.buffer(saetta_part_o_bytes(uint32_t(heads), uint32_t(capacity), uint32_t(rows)));
        part_ml_ = gpu.buffer(saetta_part_ml_bytes(uint32_t(heads), uint32_t(capacity), uint32_t(rows)));
    }
    // Row r takes its position from params[0] + r, as the reference's kernels do.
    void record(plan::Plan &plan, size_t m, const View &q, const View &keys, const View &values, const View &q_and_gate,
                const View &out, const std::vector<View> &params) const {
        if (m > rows_ || params.size() < m) throw std::runtime_error("AttentionRows::record: too many rows");
        const auto p = rows_params(m);
        const View tp = params[0];
        const gpu::Buffer po = part_o_, pml = part_ml_;
        auto launch = [=](uint32_t stage) {
            return [=](hipStream_t s) {
                check(saetta_attn_rows(s, q.ptr<float>(), keys.ptr<uint16_t>(), values.ptr<uint16_t>(), static_cast<float *>(po.get()),
                                       static_cast<float *>(pml.get()), q_and_gate.ptr<float>(), out.ptr<float>(), p,
                                       tp.ptr<saetta_token_params>(), stage),
                      "attn_rows");
            };
        };
        plan.op("attention_partial_rows_chunks", launch(SAETTA_STAGE_PARTIAL));
        plan.op("attention_reduce_rows_chunks", launch(SAETTA_STAGE_REDUCE));
    }
    void record_quant(plan::Plan &plan, size_t m, const View &q, const kv_quant::QuantRows &keys, const kv_quant::QuantRows &values,
                      const View &q_and_gate, const View &out, const std::vector<View> &params) const {
        if (m > rows_ || params.size() < m) throw std::runtime_error("AttentionRows::record_quant: too many rows");
        if (keys.bits == kv_quant::KvBits::Half) throw std::runtime_error("a half cache goes through record");
        const auto p = rows_params(m);
        const View tp = params[0];
        const gpu::Buffer po = part_o_, pml = part_ml_;
        const kv_quant::QuantRows k = keys, v = values;
        const int nbits = int(kv_quant::bits(keys.bits));
        auto launch = [=](uint32_t stage) {
            return [=](hipStream_t s) {
                check(saetta_attn_rows_quant(s, nbits, q.ptr<float>(), k.c(), v.c(), static_cast<float *>(po.get()),
                                             static_cast<float *>(pml.get()), q_and_gate.ptr<float>(), out.ptr<float>(), p,
                                             tp.ptr<saetta_token_params>(), stage),
                      "attn_rows_quant");
            };
        };
        plan.op(nbits == 8 ? "attention_partial_rows_q8" : "attention_partial_rows_q4", launch(SAETTA_STAGE_PARTIAL));
        plan.op("attention_reduce_rows", launch(SAETTA_STAGE_REDUCE));
    }

  private:
    saetta_rows_params rows_params(size_t m) const {
        return saetta_rows_params{uint32_t(heads_), uint32_t(kv_heads_), uint32_t(capacity_), 1.0f / 16.0f, uint32_t(m), uint32_t(splits_)};
    }
    size_t heads_, kv_heads_, capacity_, rows_, splits_ = 0;
    gpu::Buffer part_o_, part_ml_;
};

}  // namespace rows

namespace attention_prefill {

using FlashParams = saetta_flash_params;
inline const char *const KERNELS[2] = {"attention_fa8", "attention_fa4"};
inline const char *const DEFAULT = "attention_fa8";
constexpr size_t KEY_BLOCK = 16;

// Device memory the chunk's f16 tile images go to; the default lets the library use its own (one per
// device and stream, kept until the process ends).
struct Workspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};
inline size_t workspace_bytes(FlashParams p) { return saetta_prefill_workspace_bytes(p.pos, p.tokens, p.kv_heads); }

// out[t, h] = softmax(q[t, h] K^T * scale) V * sigmoid(gate[t, h]) over a half cache that holds
// the chunk's rows.  `kernel` picks a tile size in the reference; one gfx950 kernel serves both.
inline void encode(const gpu::Gpu &gpu, const std::string &kernel, const View &q, const View &keys, const View &values,
                   const View &q_and_gate, const View &out, FlashParams p, const Workspace &ws = {}) {
    if (kernel != KERNELS[0] && kernel != KERNELS[1]) throw std::runtime_error("no prefill attention kernel " + kernel);
    if (p.heads != p.kv_heads * 8) throw std::runtime_error(kernel + " needs 8 q heads per kv head");
    check(saetta_attn_prefill(gpu.stream(), q.ptr<uint16_t>(), keys.ptr<uint16_t>(), values.ptr<uint16_t>(), q_and_gate.ptr<float>(),
                              out.ptr<float>(), p, ws.ptr, ws.bytes),
          "attn_prefill");
}

// encode_rows2 (src/attention_prefill.rs:74-100): the reference's attention_rows2_half on the same
// buffers, its baseline in `bench`; here the same kernel as `encode`.
inline void encode_rows2(const gpu::Gpu &gpu, const View &q, const View &keys, const View &values, const View &q_and_gate,
                         const View &out, FlashParams p, const Workspace &ws = {}) {
    encode(gpu, DEFAULT, q, keys, values, q_and_gate, out, p, ws);
}

// spread (src/attention_prefill.rs:102-108): half values in about -2 .. 2, as f16 bits.
inline std::vector<uint16_t> spread(size_t n, size_t seed) {
    std::vector<uint16_t> out(n);
    for (size_t i = 0; i < n; i++) {
        const float x = float((i * 7919 + seed * 104729) % 1999) / 500.0f - 2.0f;
        const _Float16 h = static_cast<_Float16>(x);
        std::memcpy(&out[i], &h, 2);
    }
    return out;
}

// The same chunk over a quantized cache read in place (src/prefill.rs:1735-1776).
inline void encode_quant(const gpu::Gpu &gpu, const View &q, const kv_quant::QuantRows &keys, const kv_quant::QuantRows &values,
                         const View &q_and_gate, const View &out, FlashParams p, const Workspace &ws = {}) {
    if (p.heads != p.kv_heads * 8) throw std::runtime_error("prefill attention needs 8 q heads per kv head");
    check(saetta_attn_prefill_quant(gpu.stream(), int(kv_quant::bits(keys.bits)), q.ptr<uint16_t>(), keys.c(), values.c(),
                                    q_and_gate.ptr<float>(), out.ptr<float>(), p, ws.ptr, ws.bytes),
          "attn_prefill_quant");
}

}  // namespace attention_prefill

namespace attention_gemm {

constexpr size_t KEYS = SAETTA_AG_KEYS;  // src/attention_gemm.rs:28
// Query slices a chunk runs in unless SAETTA_AG_SLICES says otherwise (src/attention_gemm.rs:59-63, 83-89).
// The reference takes 2 to halve a scratch that shares the machine's one memory with the model; here 1.
constexpr size_t SLICES = 1;

inline size_t slices() {
    const char *v = std::getenv("SAETTA_AG_SLICES");
    const long n = v ? std::strtol(v, nullptr, 10) : 0;
    return n > 0 ? size_t(n) : SLICES;
}

// AttGemm (src/attention_gemm.rs:95-364): the buffers of one block for slices of up to `slice` tokens of
// a chunk, and encode.  Only the reference's default variant is built (fused, with tile sums).
struct AttGemm {
    size_t slice, rows_pad, chunk, kv_heads;
    bool fused = true, texp = true;
    // For a bench: only the first `stages` passes of each block (1, 2: scores; 3: scores and pv, no
    // outputs); 0 runs all (src/attention_gemm.rs:112-114).
    mutable uint32_t stages = 0;

    AttGemm(const gpu::Gpu &, size_t chunk_, size_t kv_heads_) : chunk(chunk_), kv_heads(kv_heads_) {
        for (const char *name : {"SAETTA_AG_FUSED", "SAETTA_AG_TEXP"}) {
            const char *v = std::getenv(name);
            if (v && std::string(v) == "0") throw std::runtime_error(std::string(name) + "=0: only the fused variant with tile sums is built");
        }
        slice = (chunk + slices() - 1) / slices();
        rows_pad = (slice * 8 + 63) / 64 * 64;
    }

    // The same as attention_prefill::encode on the same buffers; with `quant` the keys and values are read
    // from those 8- or 4-bit rows and `keys` and `values` are not read (src/attention_gemm.rs:144-188).
    void encode(const gpu::Gpu &gpu, const View &q, const View &keys, const View &values,
                const std::pair<const kv_quant::QuantRows *, const kv_quant::QuantRows *> *quant, const View &q_and_gate,
                const View &out, attention_prefill::FlashParams f) const {
        if (f.heads != f.kv_heads * 8) throw std::runtime_error("needs 8 q heads per kv head");
        if (f.tokens > chunk || f.kv_heads != kv_heads) throw std::runtime_error("AttGemm: made for another chunk or kv head count");
        int bits = 16;
        saetta_quant_rows k{const_cast<uint32_t *>(keys.ptr<uint32_t>()), nullptr, nullptr};
        saetta_quant_rows v{const_cast<uint32_t *>(values.ptr<uint32_t>()), nullptr, nullptr};
        if (quant) {
            if (quant->first->bits == kv_quant::KvBits::Half || quant->first->bits != quant->second->bits)
                throw std::runtime_error("no gemm attention for these rows");
            bits = int(kv_quant::bits(quant->first->bits));
            k = quant->first->c(), v = quant->second->c();
        }
        const size_t need = saetta_attn_gemm_workspace_bytes(f.pos, f.tokens, uint32_t(slice), f.kv_heads);
        if (workspace_.length() < need) workspace_ = gpu::Buffer(need);
        check(saetta_attn_gemm(gpu.stream(), bits, q.ptr<uint16_t>(), k, v, q_and_gate.ptr<float>(), out.ptr<float>(), f,
                               uint32_t(slice), stages, workspace_.get(), workspace_.length()),
              "attn_gemm");
    }

  private:
    mutable gpu::Buffer workspace_;
};

}  // namespace attention_gemm

namespace gpu_layers {

constexpr size_t KV_ALIGN = 128;  // src/gpu_layers.rs:199

// GpuKvCache (src/gpu_layers.rs:183-293): keys and values of one attention layer, token p in row p,
// half values or codes with their scales and biases, and the decode attention sized for the capacity.
class GpuKvCache {
  public:
    gpu::Buffer keys, values;
    std::unique_ptr<std::pair<kv_quant::QuantRows, kv_quant::QuantRows>> quant;  // Option<(QuantRows, QuantRows)>
    kv_quant::KvBits bits;
    size_t capacity;
    std::unique_ptr<attention::DecodeAttention> decode;

    GpuKvCache(const gpu::Gpu &gpu, size_t heads, size_t kv_heads, size_t head_dim, size_t capacity_,
               kv_quant::KvBits bits_ = kv_quant::KvBits::Half)
        : bits(bits_), capacity((capacity_ + KV_ALIGN - 1) / KV_ALIGN * KV_ALIGN), heads_(heads), kv_heads_(kv_heads), head_dim_(head_dim) {
        const size_t row = kv_heads * head_dim;
        decode = std::make_unique<attention::DecodeAttention>(gpu, heads, kv_heads, head_dim, capacity);
        if (bits == kv_quant::KvBits::Half) {
            keys = gpu.buffer(capacity * row * 2);
            values = gpu.buffer(capacity * row * 2);
        } else {
            quant = std::make_unique<std::pair<kv_quant::QuantRows, kv_quant::QuantRows>>(
                kv_quant::QuantRows(gpu, bits, row, capacity), kv_quant::QuantRows(gpu, bits, row, capacity));
            keys = quant->first.data;
            values = quant->second.data;
        }
    }
    // Every buffer of the cache; each holds `capacity` rows of equal size.
    std::vector<gpu::Buffer *> buffers() {
        std::vector<gpu::Buffer *> out{&keys, &values};
        if (quant) {
            for (gpu::Buffer *b : {&quant->first.scales, &quant->first.biases, &quant->second.scales, &quant->second.biases}) out.push_back(b);
        }
        return out;
    }
    // New buffers with room for `capacity_` tokens; every old row that fits is copied over.  Plans
    // recorded with the old buffers must be recorded again.
    void resize(const gpu::Gpu &gpu, size_t capacity_) {
        const size_t cap = (capacity_ + KV_ALIGN - 1) / KV_ALIGN * KV_ALIGN, rows = std::min(capacity, cap);
        for (gpu::Buffer *b : buffers()) {
            const size_t row = b->length() / capacity;
            gpu::Buffer moved = gpu.buffer(row * cap);
            hip_check(hipMemcpyAsync(moved.get(), b->get(), row * rows, hipMemcpyDeviceToDevice, gpu.stream()), "resize");
            gpu.sync();  // the old buffer goes when its last handle does
            *b = moved;
        }
        if (quant) {
            quant->first.data = keys;
            quant->second.data = values;
        }
        decode = std::make_unique<attention::DecodeAttention>(gpu, heads_, kv_heads_, head_dim_, cap);
        capacity = cap;
    }

  private:
    size_t heads_, kv_heads_, head_dim_;
};

// RowBackup (src/gpu_cache.rs:196-283): a copy of KV rows from..from + n of every attention layer;
// `restore` puts them back where they came from and frees the copy.
class RowBackup {
  public:
    size_t bytes() const {
        size_t total = 0;
        for (auto &b : parts_) total += b.length();
        return total;
    }
    void save(const gpu::Gpu &gpu, const std::vector<GpuKvCache *> &caches, size_t from, size_t n) {
        clear();
        if (n == 0) return;
        for (GpuKvCache *c : caches) {
            if (from + n > c->capacity) throw std::runtime_error("RowBackup::save: rows past the capacity");
            for (gpu::Buffer *b : c->buffers()) {
                const size_t row = b->length() / c->capacity;
                gpu::Buffer copy = gpu.buffer(n * row);
                hip_check(hipMemcpyAsync(copy.get(), static_cast<char *>(b->get()) + from * row, n * row, hipMemcpyDeviceToDevice,
                                         gpu.stream()), "RowBackup::save");
                parts_.push_back(copy);
            }
        }
        from_ = from, n_ = n;
    }
    void restore(const gpu::Gpu &gpu, const std::vector<GpuKvCache *> &caches) {
        if (parts_.empty()) return;
        size_t i = 0;
        for (GpuKvCache *c : caches) {
            for (gpu::Buffer *b : c->buffers()) {
                const size_t row = b->length() / c->capacity;
                hip_check(hipMemcpyAsync(static_cast<char *>(b->get()) + from_ * row, parts_.at(i++).get(), n_ * row,
                                         hipMemcpyDeviceToDevice, gpu.stream()), "RowBackup::restore");
            }
        }
        gpu.sync();  // the copies are freed below
        clear();
    }
    void clear() { parts_.clear(); }

  private:
    std::vector<gpu::Buffer> parts_;
    size_t from_ = 0, n_ = 0;
};

}  // namespace gpu_layers

}  // namespace saetta
