// Host-side C++ mirror of the reference's Modules/ call surface (same function names, template-parameter order
// and argument meaning), implemented on top of the C ABI in include/flexllm_hip.h.
//
// Each function drains its input stream(s) into a token-major staging buffer (undoing the reference's stream
// packing: prefill streams carry io_parallel tokens of one feature per vector, Modules/data_io.h:15-19; decode
// streams carry block_parallel block-partitioned features of one token, Modules/data_io.h:419,437), runs the
// GPU operator, and writes the result back in the packing the reference's consumer expects.
//
// Differences from the reference, all forced by the device boundary:
//  * Weights do not travel through streams: a linear layer takes a DeviceWeight that was uploaded once from
//    the row-major int8 [N][K] array (the reference's on-disk format); flexllm_adapters.h converts the reference's
//    packed weight words and KV-cache line layouts to and from that form.
//  * The int8 instantiation (qint_bit = 8, symmetric) is the W8A8 path; function names keep the reference's
//    spelling with "i8xi8" where the reference says "i4xi4".
//  * Errors throw fxhost::Error carrying flexllm_last_error() (the reference prints and returns).
#pragma once
#include <hip/hip_runtime_api.h>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>
#include <array>
#include <chrono>
#include "../../include/flexllm_hip.h"
#include "flexllm_adapters.h"
#include "stream_types.h"

namespace fxhost {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};
inline void check(int rc) {
    if (rc != FLEXLLM_OK) throw Error(std::string("flexllm: ") + flexllm_last_error());
}
inline void check_hip(hipError_t e) {
    if (e != hipSuccess) throw Error(std::string("hip: ") + hipGetErrorString(e));
}

// RAII device array
template <class T>
class DeviceArray {
public:
    DeviceArray() = default;
    explicit DeviceArray(size_t n) { resize(n); }
    explicit DeviceArray(const std::vector<T>& h) { upload(h); }
    DeviceArray(const DeviceArray&) = delete;
    DeviceArray& operator=(const DeviceArray&) = delete;
    DeviceArray(DeviceArray&& o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
    ~DeviceArray() { if (p_) (void)hipFree(p_); }
    void resize(size_t n) {
        if (p_) check_hip(hipFree(p_));
        p_ = nullptr; n_ = n;
        check_hip(hipMalloc(reinterpret_cast<void**>(&p_), (n ? n : 1) * sizeof(T)));
    }
    void upload(const std::vector<T>& h) { upload(h.data(), h.size()); }
    void upload(const T* h, size_t n) {
        if (n != n_ || !p_) resize(n);
        check_hip(hipMemcpy(p_, h, n * sizeof(T), hipMemcpyHostToDevice));
    }
    std::vector<T> download() const {
        std::vector<T> h(n_);
        check_hip(hipMemcpy(h.data(), p_, n_ * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
    T* get() const { return p_; }
    size_t size() const { return n_; }

private:
    T* p_ = nullptr;
    size_t n_ = 0;
};

// A weight matrix resident in HBM: int8 [out_dim][in_dim] row-major plus optional per-channel scales.
struct DeviceWeight {
    DeviceArray<int8_t> w;
    DeviceArray<float> scale;
    int out_dim = 0, in_dim = 0;
    DeviceWeight() = default;
    DeviceWeight(const int8_t* row_major, int n, int k, const float* s = nullptr) : out_dim(n), in_dim(k) {
        w.upload(row_major, (size_t)n * k);
        if (s) scale.upload(s, (size_t)n);
    }
};

// ---- stream <-> token-major staging ------------------------------------------------------------------
template <class T, class IS>
std::vector<T> drain_pref(IS& in, int seq_len, int dim, int io_parallel) {
    std::vector<T> x((size_t)seq_len * dim);
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int k = 0; k < dim; k++) {
            auto pack = in.read();
            for (int m = 0; m < io_parallel; m++) x[(size_t)(M * io_parallel + m) * dim + k] = (T)pack[m];
        }
    return x;
}
template <class OS, class T>
void fill_pref(OS& out, const std::vector<T>& x, int seq_len, int dim, int io_parallel) {
    using V = typename OS::value_type;
    using E = typename std::remove_reference<decltype(std::declval<V&>()[0])>::type;
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int k = 0; k < dim; k++) {
            V pack;
            for (int m = 0; m < io_parallel; m++) pack[m] = (E)x[(size_t)(M * io_parallel + m) * dim + k];
            out.write(pack);
        }
}
template <class T, class IS>
std::vector<T> drain_dec(IS& in, int dim, int block_parallel) {
    std::vector<T> x(dim);
    const int per = dim / block_parallel;
    for (int k = 0; k < per; k++) {
        auto pack = in.read();
        for (int i = 0; i < block_parallel; i++) x[(size_t)i * per + k] = (T)pack[i];
    }
    return x;
}
template <class OS, class T>
void fill_dec(OS& out, const std::vector<T>& x, int dim, int block_parallel) {
    using V = typename OS::value_type;
    using E = typename std::remove_reference<decltype(std::declval<V&>()[0])>::type;
    const int per = dim / block_parallel;
    for (int k = 0; k < per; k++) {
        V pack;
        for (int i = 0; i < block_parallel; i++) pack[i] = (E)x[(size_t)i * per + k];
        out.write(pack);
    }
}

// ======================================================================================= quant.h
// Modules/quant.h:6-13
template <int qint_bit, bool is_act_asym, int io_parallel, int max_input_dim, int max_seq_len = 1024, class IS, class OSB, class OQ>
void pref_quant_layer_fp32_qint(IS& input_stream, OSB& input_s_b_stream, OQ& output_stream, int seq_len = max_seq_len,
                                int input_dim = max_input_dim) {
    static_assert(qint_bit == 8 && !is_act_asym, "the GPU path behind this name is the symmetric int8 instantiation");
    auto x = drain_pref<float>(input_stream, seq_len, input_dim, io_parallel);
    DeviceArray<float> dx(x), ds(seq_len);
    DeviceArray<int8_t> dq((size_t)seq_len * input_dim);
    check(flexllm_quant_sym_i8(dx.get(), dq.get(), ds.get(), seq_len, input_dim, nullptr));
    auto s = ds.download();
    auto q = dq.download();
    using SV = typename OSB::value_type;
    for (int t = 0; t < seq_len; t++) { SV p; p[0] = s[t]; input_s_b_stream.write(p); }
    fill_pref(output_stream, q, seq_len, input_dim, io_parallel);
}
// Modules/quant.h:332-338
template <int qint_bit, bool is_act_asym, int block_parallel, int max_input_dim, class IS, class OSB, class OQ>
void dec_quant_layer_fp32_qint(IS& input_stream, OSB& input_s_b_stream, OQ& output_stream, int input_dim = max_input_dim) {
    static_assert((qint_bit == 8 && !is_act_asym) || is_act_asym, "symmetric int8, or asymmetric unsigned with 2..8 bits");
    auto x = drain_dec<float>(input_stream, input_dim, block_parallel);
    if constexpr (is_act_asym) {             // Modules/quant.h:382-405: scale (max-min)/(2^bits-1), zero point = min
        DeviceArray<float> dxa(x), dsa(1), dba(1);
        DeviceArray<uint8_t> dqa(input_dim);
        check(flexllm_quant_asym_u8(dxa.get(), dqa.get(), dsa.get(), dba.get(), qint_bit, 1, input_dim, nullptr));
        typename OSB::value_type pa;
        pa[0] = dsa.download()[0];
        pa[1] = dba.download()[0];
        input_s_b_stream.write(pa);
        fill_dec(output_stream, dqa.download(), input_dim, block_parallel);
        return;
    }
    DeviceArray<float> dx(x), ds(1);
    DeviceArray<int8_t> dq(input_dim);
    check(flexllm_quant_sym_i8(dx.get(), dq.get(), ds.get(), 1, input_dim, nullptr));
    typename OSB::value_type p;
    p[0] = ds.download()[0];
    input_s_b_stream.write(p);
    fill_dec(output_stream, dq.download(), input_dim, block_parallel);
}
// Modules/quant.h:115-123: weight_s_sum_stream carries one {scale} vector per output channel
template <int qint_bit, bool is_act_asym, int io_parallel, int max_output_dim, int max_seq_len = 1024, class IS, class ISB, class IW, class OS>
void pref_dequant_layer_qint_fp32(IS& input_stream, ISB& input_s_b_stream, IW& weight_s_sum_stream, OS& output_stream,
                                  int seq_len = max_seq_len, int output_dim = max_output_dim) {
    static_assert(!is_act_asym, "symmetric path");
    // the reference interleaves: per token block, io_parallel scales, then output_dim packs (and the weight
    // scales once per token block)
    std::vector<float> s(seq_len), ws(output_dim);
    std::vector<int32_t> acc((size_t)seq_len * output_dim);
    for (int M = 0; M < seq_len / io_parallel; M++) {
        for (int m = 0; m < io_parallel; m++) s[M * io_parallel + m] = input_s_b_stream.read()[0];
        for (int k = 0; k < output_dim; k++) {
            auto pack = input_stream.read();
            ws[k] = weight_s_sum_stream.read()[0];
            for (int m = 0; m < io_parallel; m++) acc[(size_t)(M * io_parallel + m) * output_dim + k] = (int32_t)pack[m];
        }
    }
    DeviceArray<int32_t> dacc(acc);
    DeviceArray<float> ds(s), dws(ws), dy((size_t)seq_len * output_dim);
    check(flexllm_dequant_i32_f32(dacc.get(), ds.get(), nullptr, dws.get(), nullptr, dy.get(), seq_len, output_dim, nullptr));
    fill_pref(output_stream, dy.download(), seq_len, output_dim, io_parallel);
}
// Modules/quant.h:470-477: weight scales arrive in groups of block_parallel*weight_parallel, lane-major
template <int qint_bit, bool is_act_asym, int block_parallel, int weight_parallel, int max_output_dim, class IS, class ISB, class IW, class OS>
void dec_dequant_layer_qint_fp32_bandwidth(IS& input_stream, ISB& input_s_b_stream, IW& weight_s_sum_stream, OS& output_stream,
                                           int output_dim = max_output_dim) {
    const auto s_b_pack = input_s_b_stream.read();
    const float s = s_b_pack[0];
    const float b = is_act_asym ? s_b_pack[is_act_asym ? 1 : 0] : 0.0f;
    const int per = output_dim / block_parallel;
    std::vector<float> ws(output_dim), wsum(output_dim);
    std::vector<int32_t> acc(output_dim);
    for (int k = 0; k < output_dim / (block_parallel * weight_parallel); k++) {
        // Modules/quant.h:491-501: weight_s[m*weight_parallel+n] belongs to lane m, step n of this group
        for (int i = 0; i < block_parallel * weight_parallel; i++) {
            const int lane = i / weight_parallel, n = i % weight_parallel;
            const auto wp = weight_s_sum_stream.read();
            ws[(size_t)lane * per + k * weight_parallel + n] = wp[0];
            if (is_act_asym) wsum[(size_t)lane * per + k * weight_parallel + n] = wp[is_act_asym ? 1 : 0];
        }
        for (int n = 0; n < weight_parallel; n++) {
            auto pack = input_stream.read();
            for (int m = 0; m < block_parallel; m++) acc[(size_t)m * per + k * weight_parallel + n] = (int32_t)pack[m];
        }
    }
    DeviceArray<int32_t> dacc(acc);
    DeviceArray<float> ds(std::vector<float>{s}), db(std::vector<float>{b}), dws(ws), dwsum(wsum), dy(output_dim);
    check(flexllm_dequant_i32_f32(dacc.get(), ds.get(), is_act_asym ? db.get() : nullptr, dws.get(),
                                  is_act_asym ? dwsum.get() : nullptr, dy.get(), 1, output_dim, nullptr));
    fill_dec(output_stream, dy.download(), output_dim, block_parallel);
}
// Modules/quant.h:252-261 (static per-layer-per-head scale)
template <int qint_bit, int io_parallel, int max_input_dim, int head_num = 1, int is_signed = true, int max_seq_len = 1024,
          int decoder_layer_num = 16, class IS, class OS>
void pref_static_sym_per_tensor_quant_layer_fp32_qint(IS& input_stream, OS& output_stream,
                                                      const float input_s[decoder_layer_num][head_num], int block_id,
                                                      int seq_len = max_seq_len, int input_dim = max_input_dim,
                                                      float mha_scale_factor = 1.0f) {
    static_assert(qint_bit == 8, "int8 path");
    auto x = drain_pref<float>(input_stream, seq_len, head_num * input_dim, io_parallel);
    DeviceArray<float> dx(x), dsc(std::vector<float>(input_s[block_id], input_s[block_id] + head_num));
    DeviceArray<int8_t> dq(x.size());
    check(flexllm_static_quant_i8(dx.get(), dq.get(), dsc.get(), mha_scale_factor, is_signed, seq_len, head_num, input_dim, nullptr));
    auto q = dq.download();
    if (is_signed) fill_pref(output_stream, q, seq_len, head_num * input_dim, io_parallel);
    else {
        std::vector<uint8_t> u(q.begin(), q.end());
        fill_pref(output_stream, u, seq_len, head_num * input_dim, io_parallel);
    }
}

// ======================================================================================= Linear_Layer.h
// Modules/Linear_Layer.h:293-301 with the weight stream replaced by a resident DeviceWeight
template <int io_parallel, int weight_parallel, int max_input_dim = 2048, int max_log2_input_dim = 11, int max_output_dim = 2048,
          int max_seq_len = 1024, bool is_uint_input = false, class IS, class OS>
void pref_Linear_Layer_i8xi8(IS& input_seq, const DeviceWeight& weight, OS& output_seq, int seq_len = max_seq_len,
                             int input_dim = max_input_dim, int output_dim = max_output_dim) {
    static_assert(!is_uint_input, "signed activations");
    auto a = drain_pref<int8_t>(input_seq, seq_len, input_dim, io_parallel);
    DeviceArray<int8_t> da(a);
    DeviceArray<int32_t> dc((size_t)seq_len * output_dim);
    check(flexllm_linear_i8_gemm(da.get(), weight.w.get(), dc.get(), seq_len, input_dim, output_dim, nullptr));
    fill_pref(output_seq, dc.download(), seq_len, output_dim, io_parallel);
}
// Modules/Linear_Layer.h:862-869; the output is block-partitioned over block_parallel lanes like the input
template <int block_parallel, int weight_parallel, int max_input_dim = 2048, int max_log2_input_dim = 11, int max_output_dim = 2048,
          bool is_uint_input = false, class IS, class OS>
void dec_Linear_Layer_i8xi8(IS& input_seq, const DeviceWeight& weight, OS& output_seq, int input_dim = max_input_dim,
                            int output_dim = max_output_dim) {
    static_assert(!is_uint_input, "signed activations");
    auto x = drain_dec<int8_t>(input_seq, input_dim, block_parallel);
    DeviceArray<int8_t> dx(x);
    DeviceArray<int32_t> dc(output_dim);
    check(flexllm_linear_i8_gemv(dx.get(), weight.w.get(), dc.get(), input_dim, output_dim, nullptr));
    fill_dec(output_seq, dc.download(), output_dim, block_parallel);
}
// A 4-bit weight matrix resident in HBM: values -8..7, two per byte along the input dimension (low nibble = even
// index), from the row-major one-value-per-byte form the testbenches build (q_weight_val, …_tb.cpp:184).
struct DeviceWeight4 {
    DeviceArray<uint8_t> w4;
    int out_dim = 0, in_dim = 0;
    DeviceWeight4() = default;
    DeviceWeight4(const int8_t* row_major, int n, int k) : out_dim(n), in_dim(k) {
        std::vector<uint8_t> p((size_t)n * k / 2);
        for (size_t i = 0; i < p.size(); i++) p[i] = (uint8_t)((row_major[2 * i] & 0xF) | ((row_major[2 * i + 1] & 0xF) << 4));
        w4.upload(p);
    }
};
// Modules/Linear_Layer.h:862-869 (is_uint_input = true: unsigned 4-bit activations), weight streams replaced by
// a resident DeviceWeight4
template <int block_parallel, int weight_parallel, int max_input_dim = 2048, int max_log2_input_dim = 11, int max_output_dim = 2048,
          bool is_uint_input = false, class IS, class OS>
void dec_Linear_Layer_i4xi4(IS& input_seq, const DeviceWeight4& weight, OS& output_seq, int input_dim = max_input_dim,
                            int output_dim = max_output_dim) {
    static_assert(is_uint_input, "the W4A4 path has unsigned (asymmetric) activations");
    auto x = drain_dec<uint8_t>(input_seq, input_dim, block_parallel);
    std::vector<uint8_t> x4(input_dim / 2);
    for (int i = 0; i < input_dim / 2; i++) x4[i] = (uint8_t)((x[2 * i] & 0xF) | ((x[2 * i + 1] & 0xF) << 4));
    DeviceArray<uint8_t> dx(x4);
    DeviceArray<int32_t> dc(output_dim);
    check(flexllm_linear_u4i4_gemv(dx.get(), weight.w4.get(), dc.get(), input_dim, output_dim, nullptr));
    fill_dec(output_seq, dc.download(), output_dim, block_parallel);
}
// Modules/Linear_Layer.h:293-301 (is_uint_input = true), the weight stream replaced by a resident DeviceWeight4: seq_len
// tokens of unsigned 4-bit activations in the prefill packing -> int32 accumulators in the same packing
template <int io_parallel, int weight_parallel, int max_input_dim = 2048, int max_log2_input_dim = 11, int max_output_dim = 2048,
          int max_seq_len = 1024, bool is_uint_input = false, class IS, class OS>
void pref_Linear_Layer_i4xi4(IS& input_seq, const DeviceWeight4& weight, OS& output_seq, int seq_len = max_seq_len,
                             int input_dim = max_input_dim, int output_dim = max_output_dim) {
    static_assert(is_uint_input, "the W4A4 path has unsigned (asymmetric) activations");
    auto a = drain_pref<uint8_t>(input_seq, seq_len, input_dim, io_parallel);
    std::vector<uint8_t> a4(a.size() / 2);
    for (size_t i = 0; i < a4.size(); i++) a4[i] = (uint8_t)((a[2 * i] & 0xF) | ((a[2 * i + 1] & 0xF) << 4));
    DeviceArray<uint8_t> da(a4);
    DeviceArray<int32_t> dc((size_t)seq_len * output_dim);
    check(flexllm_linear_u4i4_gemm(da.get(), weight.w4.get(), dc.get(), seq_len, input_dim, output_dim, nullptr));
    fill_pref(output_seq, dc.download(), seq_len, output_dim, io_parallel);
}
// Modules/Linear_Layer.h:612-617 / :1103-1108
template <int io_parallel, int io_hidden_dim, int max_seq_len = 1024, class IA, class IB, class OS>
void pref_Gate_Layer_fp32xfp32(IA& input_seq, IB& gate_seq, OS& output_seq, int seq_len = max_seq_len) {
    for (int i = 0; i < seq_len / io_parallel * io_hidden_dim; i++) {
        auto a = input_seq.read();
        auto b = gate_seq.read();
        typename OS::value_type o;
        for (int m = 0; m < io_parallel; m++) o[m] = a[m] * b[m];
        output_seq.write(o);
    }
}
template <int block_parallel, int max_hidden_dim = 2048, class IA, class IB, class OS>
void dec_Gate_Layer_fp32xfp32(IA& input_seq, IB& gate_seq, OS& output_seq, int io_hidden_dim = max_hidden_dim) {
    for (int i = 0; i < io_hidden_dim / block_parallel; i++) {
        auto a = input_seq.read();
        auto b = gate_seq.read();
        typename OS::value_type o;
        for (int m = 0; m < block_parallel; m++) o[m] = a[m] * b[m];
        output_seq.write(o);
    }
}

// ======================================================================================= FHT.h
// Modules/FHT.h:7-13
template <typename T, int io_parallel, int io_hidden_dim = 2048, int log2_io_hidden_dim = 11, int max_seq_len = 1024, class IS, class OS>
void pref_FHT(IS& data_in, OS& data_out, int seq_len = max_seq_len, const T scale_factor = 1.0) {
    static_assert(std::is_same<T, float>::value && (1 << log2_io_hidden_dim) == io_hidden_dim, "fp32, power-of-two length");
    auto x = drain_pref<float>(data_in, seq_len, io_hidden_dim, io_parallel);
    DeviceArray<float> dx(x);
    check(flexllm_fht_f32(dx.get(), dx.get(), seq_len, io_hidden_dim, scale_factor, nullptr));
    fill_pref(data_out, dx.download(), seq_len, io_hidden_dim, io_parallel);
}
// Modules/FHT.h:69-74
template <typename T, int block_parallel, int io_hidden_dim = 8192, int log2_io_hidden_dim = 13, class IS, class OS>
void dec_FHT(IS& data_in, OS& data_out, const T scale_factor = 1.0) {
    static_assert(std::is_same<T, float>::value && (1 << log2_io_hidden_dim) == io_hidden_dim, "fp32, power-of-two length");
    auto x = drain_dec<float>(data_in, io_hidden_dim, block_parallel);
    DeviceArray<float> dx(x);
    check(flexllm_fht_f32(dx.get(), dx.get(), 1, io_hidden_dim, scale_factor, nullptr));
    fill_dec(data_out, dx.download(), io_hidden_dim, block_parallel);
}

// ======================================================================================= LayerNorm.h
// Modules/LayerNorm.h:28-36 (RMSNorm, beta disabled); gamma arrives one value per read
template <typename T, int io_parallel, int max_hidden_dim = 2048, int max_seq_len = 1024, bool enble_beta = false, bool is_versal = false,
          class IS, class IG, class OS>
void pref_Layer_Norm(IS& input_stream, IG& gamma_beta_stream, OS& output_stream, int seq_len = max_seq_len,
                     int io_hidden_dim = max_hidden_dim, const T eps = 0.00001) {
    static_assert(!enble_beta, "RMSNorm path");
    std::vector<float> g(io_hidden_dim);
    for (int k = 0; k < io_hidden_dim; k++) g[k] = gamma_beta_stream.read();
    auto x = drain_pref<float>(input_stream, seq_len, io_hidden_dim, io_parallel);
    DeviceArray<float> dx(x), dg(g), dy(x.size());
    check(flexllm_rmsnorm_f32(dx.get(), dg.get(), dy.get(), seq_len, io_hidden_dim, eps, nullptr));
    fill_pref(output_stream, dy.download(), seq_len, io_hidden_dim, io_parallel);
}
// Modules/LayerNorm.h:210-217; gamma arrives block-partitioned like the activations
template <typename T, int block_parallel, int max_hidden_dim = 2048, bool enble_beta = false, bool is_versal = false, class IS, class IG,
          class OS>
void dec_Layer_Norm(IS& input_stream, IG& gamma_beta_stream, OS& output_stream, int io_hidden_dim = max_hidden_dim,
                    const T eps = 0.00001) {
    static_assert(!enble_beta, "RMSNorm path");
    auto g = drain_dec<float>(gamma_beta_stream, io_hidden_dim, block_parallel);
    auto x = drain_dec<float>(input_stream, io_hidden_dim, block_parallel);
    DeviceArray<float> dx(x), dg(g), dy(x.size());
    check(flexllm_rmsnorm_f32(dx.get(), dg.get(), dy.get(), 1, io_hidden_dim, eps, nullptr));
    fill_dec(output_stream, dy.download(), io_hidden_dim, block_parallel);
}

// ======================================================================================= RoPE.h
// Modules/RoPE.h:8-15: stream order per token block is head-major, head_dim features per head
template <typename T, int io_parallel, int io_hidden_dim = 64, int max_head_num = 32, int max_seq_Len = 1024, class IS, class OS>
void pref_RoPE_layer(IS& input_stream, OS& output_stream, const T PE_sin[max_seq_Len][io_hidden_dim / 2],
                     const T PE_cos[max_seq_Len][io_hidden_dim / 2], int head_num = max_head_num, int seq_len = max_seq_Len) {
    auto x = drain_pref<float>(input_stream, seq_len, head_num * io_hidden_dim, io_parallel);
    DeviceArray<float> dx(x), dy(x.size());
    DeviceArray<float> ds, dc;
    ds.upload(&PE_sin[0][0], (size_t)max_seq_Len * (io_hidden_dim / 2));
    dc.upload(&PE_cos[0][0], (size_t)max_seq_Len * (io_hidden_dim / 2));
    check(flexllm_rope_f32(dx.get(), dy.get(), ds.get(), dc.get(), seq_len, head_num, io_hidden_dim, 0, nullptr));
    fill_pref(output_stream, dy.download(), seq_len, head_num * io_hidden_dim, io_parallel);
}

// ======================================================================================= Swish.h / Residual_Layer.h / Softmax.h
// Modules/Swish.h:5-10
template <typename T, int io_parallel, int max_hidden_dim = 8192, int max_seq_len = 1024, class IS, class OS>
void pref_Swish(IS& input_stream, OS& output_stream, int seq_len = max_seq_len, int io_hidden_dim = max_hidden_dim) {
    auto x = drain_pref<float>(input_stream, seq_len, io_hidden_dim, io_parallel);
    DeviceArray<float> dx(x);
    check(flexllm_swish_f32(dx.get(), dx.get(), x.size(), nullptr));
    fill_pref(output_stream, dx.download(), seq_len, io_hidden_dim, io_parallel);
}
// Modules/Swish.h:26-30
template <typename T, int block_parallel, int max_hidden_dim = 8192, class IS, class OS>
void dec_Swish(IS& input_stream, OS& output_stream, int io_hidden_dim = max_hidden_dim) {
    auto x = drain_dec<float>(input_stream, io_hidden_dim, block_parallel);
    DeviceArray<float> dx(x);
    check(flexllm_swish_f32(dx.get(), dx.get(), x.size(), nullptr));
    fill_dec(output_stream, dx.download(), io_hidden_dim, block_parallel);
}
// Modules/Residual_Layer.h:47-53
template <typename T, int io_parallel, int io_hidden_dim = 2048, int max_seq_len = 1024, class IA, class IB, class OS>
void pref_Residual_Layer(IA& input_stream, IB& residual_stream, OS& output_stream, int seq_len = max_seq_len) {
    auto a = drain_pref<float>(input_stream, seq_len, io_hidden_dim, io_parallel);
    auto b = drain_pref<float>(residual_stream, seq_len, io_hidden_dim, io_parallel);
    DeviceArray<float> da(a), db(b);
    check(flexllm_residual_add_f32(da.get(), db.get(), da.get(), a.size(), nullptr));
    fill_pref(output_stream, da.download(), seq_len, io_hidden_dim, io_parallel);
}
// Modules/Residual_Layer.h:69-75
template <typename T, int block_parallel, int max_hidden_dim = 2048, class IA, class IB, class OS>
void dec_Residual_Layer(IA& input_stream, IB& residual_stream, OS& output_stream, int io_hidden_dim = max_hidden_dim) {
    auto a = drain_dec<float>(input_stream, io_hidden_dim, block_parallel);
    auto b = drain_dec<float>(residual_stream, io_hidden_dim, block_parallel);
    DeviceArray<float> da(a), db(b);
    check(flexllm_residual_add_f32(da.get(), db.get(), da.get(), a.size(), nullptr));
    fill_dec(output_stream, da.download(), io_hidden_dim, block_parallel);
}
// Modules/Softmax.h:6-12: per token block, head_num rows of io_hidden_dim scores per token
template <typename T, int io_parallel, int max_hidden_dim = 2048, int max_seq_len = 1024, int head_num = 1, bool enable_scale = false,
          bool enable_sub_max = true, bool is_versal = false, class IS, class OS>
void pref_Softmax(IS& input_stream, OS& output_stream, int seq_len = max_seq_len, int io_hidden_dim = max_hidden_dim,
                  const T scale_factor = 1.0) {
    static_assert(!enable_scale && enable_sub_max, "the configuration the shipped graphs use");
    auto x = drain_pref<float>(input_stream, seq_len, head_num * io_hidden_dim, io_parallel);   // [token][head][dim]
    DeviceArray<float> dx(x);
    check(flexllm_softmax_f32(dx.get(), dx.get(), seq_len * head_num, io_hidden_dim, nullptr));
    fill_pref(output_stream, dx.download(), seq_len, head_num * io_hidden_dim, io_parallel);
}

// ======================================================================================= decode-side attention modules
// Head-parallel decode streams carry head_parallel heads per vector: lane m of step H is head m*(head_num/HP) + H
// (Modules/quant.h:736, :793), dim values per head in sequence.
template <class T, class IS>
std::vector<T> drain_heads(IS& in, int head_num, int dim, int head_parallel) {
    std::vector<T> x((size_t)head_num * dim);
    const int per = head_num / head_parallel;
    for (int H = 0; H < per; H++)
        for (int k = 0; k < dim; k++) {
            auto pack = in.read();
            for (int m = 0; m < head_parallel; m++) x[(size_t)(m * per + H) * dim + k] = (T)pack[m];
        }
    return x;
}
template <class OS, class T>
void fill_heads(OS& out, const std::vector<T>& x, int head_num, int dim, int head_parallel) {
    using V = typename OS::value_type;
    using E = typename std::remove_reference<decltype(std::declval<V&>()[0])>::type;
    const int per = head_num / head_parallel;
    for (int H = 0; H < per; H++)
        for (int k = 0; k < dim; k++) {
            V pack;
            for (int m = 0; m < head_parallel; m++) pack[m] = (E)x[(size_t)(m * per + H) * dim + k];
            out.write(pack);
        }
}
// Modules/RoPE.h:96-103
template <typename T, int head_parallel, int io_hidden_dim = 64, int max_head_num = 32, int max_sum_seq_len = 2048, class IS, class OS>
void dec_RoPE_layer(IS& input_stream, OS& output_stream, const T PE_sin[max_sum_seq_len][io_hidden_dim / 2],
                    const T PE_cos[max_sum_seq_len][io_hidden_dim / 2], int head_num = max_head_num, int seq_id = 0) {
    auto x = drain_heads<float>(input_stream, head_num, io_hidden_dim, head_parallel);
    DeviceArray<float> dx(x), dy(x.size()), ds, dc;
    // only the row of this position is needed on the device; it is passed as a one-row table at position 0
    ds.upload(&PE_sin[seq_id][0], (size_t)(io_hidden_dim / 2));
    dc.upload(&PE_cos[seq_id][0], (size_t)(io_hidden_dim / 2));
    check(flexllm_rope_f32(dx.get(), dy.get(), ds.get(), dc.get(), 1, head_num, io_hidden_dim, 0, nullptr));
    fill_heads(output_stream, dy.download(), head_num, io_hidden_dim, head_parallel);
}
// Modules/Softmax.h:456-461: one row of io_hidden_dim scores per head
template <typename T, int head_parallel, int max_hidden_dim = 2048, int head_num = 1, bool enable_scale = false, bool enable_sub_max = true,
          bool is_versal = false, class IS, class OS>
void dec_MHA_Softmax(IS& input_stream, OS& output_stream, int io_hidden_dim = max_hidden_dim, const T scale_factor = 1.0) {
    static_assert(!enable_scale && enable_sub_max, "the configuration the shipped graphs use");
    auto x = drain_heads<float>(input_stream, head_num, io_hidden_dim, head_parallel);
    DeviceArray<float> dx(x);
    check(flexllm_softmax_f32(dx.get(), dx.get(), head_num, io_hidden_dim, nullptr));
    fill_heads(output_stream, dx.download(), head_num, io_hidden_dim, head_parallel);
}
// Modules/quant.h:716-724
template <int qint_bit, int head_parallel, int max_input_dim, int head_num = 1, bool is_signed = true, int decoder_layer_num = 16,
          class IS, class OS>
void dec_MHA_static_sym_per_tensor_quant_layer_fp32_qint(IS& input_stream, OS& output_stream,
                                                         const float input_s[decoder_layer_num][head_num], int block_id,
                                                         int input_dim = max_input_dim, float mha_scale_factor = 1.0f) {
    static_assert(qint_bit == 8, "int8 path");
    auto x = drain_heads<float>(input_stream, head_num, input_dim, head_parallel);
    DeviceArray<float> dx(x), dsc(std::vector<float>(input_s[block_id], input_s[block_id] + head_num));
    DeviceArray<int8_t> dq(x.size());
    check(flexllm_static_quant_i8(dx.get(), dq.get(), dsc.get(), mha_scale_factor, is_signed, 1, head_num, input_dim, nullptr));
    auto q = dq.download();
    if (is_signed) fill_heads(output_stream, q, head_num, input_dim, head_parallel);
    else fill_heads(output_stream, std::vector<uint8_t>(q.begin(), q.end()), head_num, input_dim, head_parallel);
}
// Modules/quant.h:758-766: act head a_H = m*(act_heads/HP) + h, weight head a_H / (act_heads / weight_heads)
template <int qint_bit, int head_parallel, int max_output_dim, int act_head_num = 1, int weight_head_num = 1, int decoder_layer_num = 16,
          class IS, class OS>
void dec_MHA_static_sym_per_tensor_dequant_layer_qint_fp32(IS& input_stream, OS& output_stream,
                                                           const float input_s[decoder_layer_num][act_head_num],
                                                           const float weight_s[decoder_layer_num][weight_head_num], int block_id,
                                                           int output_dim = max_output_dim) {
    auto acc = drain_heads<int32_t>(input_stream, act_head_num, output_dim, head_parallel);
    DeviceArray<int32_t> dacc(acc);
    DeviceArray<float> das(std::vector<float>(input_s[block_id], input_s[block_id] + act_head_num)),
        dws(std::vector<float>(weight_s[block_id], weight_s[block_id] + weight_head_num)), dy(acc.size());
    check(flexllm_static_dequant_i32_f32(dacc.get(), dy.get(), das.get(), dws.get(), 1, act_head_num, weight_head_num, output_dim, nullptr));
    fill_heads(output_stream, dy.download(), act_head_num, output_dim, head_parallel);
}
// Modules/quant.h:296-305: per token block, heads in order h*(act/weight)+g, output_dim values each
template <int qint_bit, int io_parallel, int max_output_dim, int act_head_num = 1, int weight_head_num = 1, int max_seq_len = 1024,
          int decoder_layer_num = 16, class IS, class OS>
void pref_static_sym_per_tensor_dequant_layer_qint_fp32(IS& input_stream, OS& output_stream,
                                                        const float input_s[decoder_layer_num][act_head_num],
                                                        const float weight_s[decoder_layer_num][weight_head_num], int block_id,
                                                        int seq_len = max_seq_len, int output_dim = max_output_dim) {
    auto acc = drain_pref<int32_t>(input_stream, seq_len, act_head_num * output_dim, io_parallel);      // [token][head][dim]
    DeviceArray<int32_t> dacc(acc);
    DeviceArray<float> das(std::vector<float>(input_s[block_id], input_s[block_id] + act_head_num)),
        dws(std::vector<float>(weight_s[block_id], weight_s[block_id] + weight_head_num)), dy(acc.size());
    check(flexllm_static_dequant_i32_f32(dacc.get(), dy.get(), das.get(), dws.get(), seq_len, act_head_num, weight_head_num, output_dim, nullptr));
    fill_pref(output_stream, dy.download(), seq_len, act_head_num * output_dim, io_parallel);
}
// Modules/MHA.h:246-251: entries with key index k beyond the token's own position become -1e32.  A selection without
// arithmetic: done while re-packing the stream.
template <typename T, int io_parallel, int max_hidden_dim = 2048, int max_seq_len = 1024, int head_num = 1, class IS, class OS>
void pref_causal_mask_template(IS& input_stream, OS& output_stream, int seq_len = max_seq_len, int io_hidden_dim = max_hidden_dim) {
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int H = 0; H < head_num; H++)
            for (int k = 0; k < io_hidden_dim; k++) {
                auto in = input_stream.read();
                typename OS::value_type o;
                for (int i = 0; i < io_parallel; i++) o[i] = k <= M * io_parallel + i ? (T)in[i] : (T)-1e32;
                output_stream.write(o);
            }
}
// Modules/MHA.h:189-194.  The key stream carries, per token block M and query head H, the keys of that head's KV head in
// blocks of K_parallel keys, feature-major inside a block (the cache manager's read order, Modules/MHA.h:96-106); the keys
// are the same in every token block, so the first block's copy is kept and the repeats are read and dropped.
template <int io_parallel, int K_parallel, int mha_head_num, int mha_head_dim = 64, int log2_mha_head_dim = 6, int max_seq_len = 1024,
          bool is_uint_input = false, class IS, class IK, class OS>
void pref_MHA_i8xi8_qxk_template(IS& input_seq, IK& weight_loader, OS& output_seq, int seq_len = max_seq_len) {
    static_assert(!is_uint_input, "queries are signed");
    const int hd = mha_head_dim;
    std::vector<int8_t> q((size_t)mha_head_num * seq_len * hd), kk((size_t)mha_head_num * seq_len * hd);     // [head][token][d]
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int H = 0; H < mha_head_num; H++) {
            for (int k = 0; k < hd; k++) {
                auto pack = input_seq.read();
                for (int m = 0; m < io_parallel; m++) q[((size_t)H * seq_len + M * io_parallel + m) * hd + k] = (int8_t)(int)pack[m];
            }
            for (int N = 0; N < seq_len / K_parallel; N++)
                for (int k = 0; k < hd; k++) {
                    auto kp = weight_loader.read();
                    if (M == 0)
                        for (int j = 0; j < K_parallel; j++) kk[((size_t)H * seq_len + N * K_parallel + j) * hd + k] = (int8_t)(int)kp[j];
                }
        }
    DeviceArray<int8_t> dq(q), dk(kk);
    DeviceArray<int32_t> dacc((size_t)mha_head_num * seq_len * seq_len);
    for (int H = 0; H < mha_head_num; H++)
        check(flexllm_linear_i8_gemm(dq.get() + (size_t)H * seq_len * hd, dk.get() + (size_t)H * seq_len * hd,
                                     dacc.get() + (size_t)H * seq_len * seq_len, seq_len, hd, seq_len, nullptr));
    auto acc = dacc.download();
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int H = 0; H < mha_head_num; H++)
            for (int n = 0; n < seq_len; n++) {
                typename OS::value_type o;
                for (int m = 0; m < io_parallel; m++) o[m] = acc[((size_t)H * seq_len + M * io_parallel + m) * seq_len + n];
                output_seq.write(o);
            }
}
// Modules/MHA.h:339-344: probabilities [token][head][key] (unsigned when is_uint_input), V blocks of V_parallel channels,
// key-major inside a block, repeated per token block like the keys above.
template <int io_parallel, int V_parallel, int mha_head_num, int mha_head_dim = 64, int max_seq_len = 1024, int log2_max_seq_len = 10,
          bool is_uint_input = false, class IS, class IV, class OS>
void pref_MHA_i8xi8_axv_template(IS& input_seq, IV& weight_loader, OS& output_seq, int seq_len = max_seq_len) {
    static_assert(is_uint_input, "the probabilities are unsigned 8-bit");
    const int hd = mha_head_dim;
    std::vector<uint8_t> p((size_t)mha_head_num * seq_len * seq_len);                                       // [head][token][key]
    std::vector<int8_t> vt((size_t)mha_head_num * hd * seq_len);                                            // [head][channel][key]
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int H = 0; H < mha_head_num; H++) {
            for (int k = 0; k < seq_len; k++) {
                auto pack = input_seq.read();
                for (int m = 0; m < io_parallel; m++) p[((size_t)H * seq_len + M * io_parallel + m) * seq_len + k] = (uint8_t)(int)pack[m];
            }
            for (int N = 0; N < hd / V_parallel; N++)
                for (int k = 0; k < seq_len; k++) {
                    auto vp = weight_loader.read();
                    if (M == 0)
                        for (int j = 0; j < V_parallel; j++) vt[((size_t)H * hd + N * V_parallel + j) * seq_len + k] = (int8_t)(int)vp[j];
                }
        }
    DeviceArray<uint8_t> dp(p);
    DeviceArray<int8_t> dv(vt);
    DeviceArray<int32_t> dacc((size_t)mha_head_num * seq_len * hd);
    for (int H = 0; H < mha_head_num; H++)
        check(flexllm_linear_u8i8_gemm(dp.get() + (size_t)H * seq_len * seq_len, dv.get() + (size_t)H * hd * seq_len,
                                       dacc.get() + (size_t)H * seq_len * hd, seq_len, seq_len, hd, nullptr));
    auto acc = dacc.download();
    for (int M = 0; M < seq_len / io_parallel; M++)
        for (int H = 0; H < mha_head_num; H++)
            for (int n = 0; n < hd; n++) {
                typename OS::value_type o;
                for (int m = 0; m < io_parallel; m++) o[m] = acc[((size_t)H * seq_len + M * io_parallel + m) * hd + n];
                output_seq.write(o);
            }
}
// Modules/MHA.h:615-620: one query per head; lane i's key stream carries, for each of its heads H, the keys in blocks of
// K_parallel (the last block padded with whatever the cache line holds), feature-major inside a block.  The scores of the
// padded keys are produced too, as in the reference (dec_quant_a_discard_template drops them afterwards).
template <int head_parallel, int K_parallel, int mha_head_num, int mha_head_dim = 64, int log2_mha_head_dim = 6, int max_sum_seq_len = 2048,
          bool is_uint_input = false, class IS, class IKS, class OS>
void dec_MHA_i8xi8_qxk_template(IS& input_seq, IKS& weight_loaders, OS& output_seq, int seq_len) {
    static_assert(!is_uint_input, "queries are signed");
    const int hd = mha_head_dim, per = mha_head_num / head_parallel;
    const int padded = (seq_len + K_parallel - 1) / K_parallel * K_parallel;
    auto q = drain_heads<int8_t>(input_seq, mha_head_num, hd, head_parallel);                               // [head][d]
    std::vector<int8_t> kk((size_t)mha_head_num * padded * hd);                                             // [head][key][d]
    for (int H = 0; H < per; H++)
        for (int N = 0; N < padded / K_parallel; N++)
            for (int k = 0; k < hd; k++)
                for (int i = 0; i < head_parallel; i++) {
                    auto kp = weight_loaders[i].read();
                    for (int j = 0; j < K_parallel; j++) kk[((size_t)(i * per + H) * padded + N * K_parallel + j) * hd + k] = (int8_t)(int)kp[j];
                }
    DeviceArray<int8_t> dq(q), dk(kk);
    DeviceArray<int32_t> dacc((size_t)mha_head_num * padded);
    for (int h = 0; h < mha_head_num; h++)
        check(flexllm_linear_i8_gemv(dq.get() + (size_t)h * hd, dk.get() + (size_t)h * padded * hd, dacc.get() + (size_t)h * padded, hd, padded, nullptr));
    fill_heads(output_seq, dacc.download(), mha_head_num, padded, head_parallel);
}
// Modules/MHA.h:854-859
template <int head_parallel, int V_parallel, int mha_head_num, int mha_head_dim = 64, int max_sum_seq_len = 2048, int log2_max_sum_seq_len = 11,
          bool is_uint_input = false, class IS, class IVS, class OS>
void dec_MHA_i8xi8_axv_template(IS& input_seq, IVS& weight_loaders, OS& output_seq, int seq_len) {
    static_assert(is_uint_input, "the probabilities are unsigned 8-bit");
    const int hd = mha_head_dim, per = mha_head_num / head_parallel;
    const int kpad = (seq_len + 15) / 16 * 16;                                                               // the product wants k % 16 == 0
    std::vector<uint8_t> p((size_t)mha_head_num * kpad, 0);                                                  // [head][key], zero padding
    std::vector<int8_t> vt((size_t)mha_head_num * hd * kpad, 0);                                             // [head][channel][key]
    for (int H = 0; H < per; H++) {
        for (int k = 0; k < seq_len; k++) {
            auto pack = input_seq.read();
            for (int i = 0; i < head_parallel; i++) p[(size_t)(i * per + H) * kpad + k] = (uint8_t)(int)pack[i];
        }
        for (int N = 0; N < hd / V_parallel; N++)
            for (int k = 0; k < seq_len; k++)
                for (int i = 0; i < head_parallel; i++) {
                    auto vp = weight_loaders[i].read();
                    for (int j = 0; j < V_parallel; j++) vt[((size_t)(i * per + H) * hd + N * V_parallel + j) * kpad + k] = (int8_t)(int)vp[j];
                }
    }
    DeviceArray<uint8_t> dp(p);
    DeviceArray<int8_t> dv(vt);
    DeviceArray<int32_t> dacc((size_t)mha_head_num * hd);
    for (int h = 0; h < mha_head_num; h++)
        check(flexllm_linear_u8i8_gemm(dp.get() + (size_t)h * kpad, dv.get() + (size_t)h * hd * kpad, dacc.get() + (size_t)h * hd, 1, kpad, hd, nullptr));
    fill_heads(output_seq, dacc.download(), mha_head_num, hd, head_parallel);
}

// ======================================================================================= launcher
// tapa::invoke-shaped launcher: `top` is called with the remaining arguments and the elapsed time is returned in
// nanoseconds, as tapa::invoke does (SpinQuant_Llama_32_1B/MHA_i8xi8_decoding_tb.cpp:241-252).  The bitstream argument is
// kept for the call shape: "hip" (or an empty string, the reference's software-simulation spelling) runs on the GPU, any
// other value is refused - there is no other backend.  The *_mmap(...) wrappers of the reference only tell TAPA the copy
// direction; here they pass the host vectors through.
template <class T> T& read_only_mmap(T& v) { return v; }
template <class T> const T& read_only_mmap(const T& v) { return v; }
template <class T> T& write_only_mmap(T& v) { return v; }
template <class T> T& read_write_mmap(T& v) { return v; }
template <class T, size_t N> T (&read_only_mmaps(T (&v)[N]))[N] { return v; }
template <class T, size_t N> T (&read_write_mmaps(T (&v)[N]))[N] { return v; }
template <class F, class... A>
int64_t invoke(F&& top, const std::string& bitstream, A&&... args) {
    if (!bitstream.empty() && bitstream != "hip") throw Error("fxhost::invoke: unknown bitstream '" + bitstream + "' (only \"hip\")");
    check_hip(hipDeviceSynchronize());
    const auto t0 = std::chrono::steady_clock::now();
    top(std::forward<A>(args)...);
    check_hip(hipDeviceSynchronize());
    return (int64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
}

// ======================================================================================= MHA_i8xi8.h tops
// MHA_i8xi8_Prefilling_tb (SpinQuant_Llama_32_1B/MHA_i8xi8.h:369-427) for ONE layer: q_mmap/k_mmap/v_mmap and
// o_mmap use the prefill packing [(token/TP)*dim + feature][token%TP]; scales are that layer's rows of
// Q_s/K_s/V_s/A_s.  Returns the kernel time in ns like tapa::invoke.
template <int TP, int q_heads, int kv_heads, int head_dim, class VF>
int64_t MHA_i8xi8_Prefilling_layer(const std::vector<VF>& q_mmap, const std::vector<VF>& k_mmap, const std::vector<VF>& v_mmap,
                                   std::vector<VF>& o_mmap, const float* Q_s, const float* K_s, const float* V_s,
                                   const float* A_s, int seq_len, float sqrt_head_dim) {
    const int H = q_heads * head_dim, KV = kv_heads * head_dim;
    auto unpack = [&](const std::vector<VF>& mm, int dim) {
        std::vector<float> x((size_t)seq_len * dim);
        for (int t = 0; t < seq_len; t++)
            for (int j = 0; j < dim; j++) x[(size_t)t * dim + j] = mm[(size_t)(t / TP) * dim + j][t % TP];
        return x;
    };
    DeviceArray<float> dq(unpack(q_mmap, H)), dk(unpack(k_mmap, KV)), dv(unpack(v_mmap, KV)), dout((size_t)seq_len * H);
    DeviceArray<float> dqs(std::vector<float>(Q_s, Q_s + q_heads)), dks(std::vector<float>(K_s, K_s + kv_heads)),
        dvs(std::vector<float>(V_s, V_s + kv_heads)), das(std::vector<float>(A_s, A_s + q_heads));
    const int max_pos = (seq_len + 63) / 64 * 64;
    DeviceArray<int8_t> q8((size_t)seq_len * H), kc((size_t)kv_heads * max_pos * head_dim), vc((size_t)kv_heads * max_pos * head_dim);
    flexllm_mha_scales sc{dqs.get(), dks.get(), dvs.get(), das.get()};
    hipEvent_t e0, e1;
    check_hip(hipEventCreate(&e0)); check_hip(hipEventCreate(&e1));
    check_hip(hipEventRecord(e0, nullptr));
    check(flexllm_static_quant_i8(dq.get(), q8.get(), dqs.get(), sqrt_head_dim, 1, seq_len, q_heads, head_dim, nullptr));
    check(flexllm_kv_append_i8(dk.get(), dv.get(), kc.get(), vc.get(), &sc, seq_len, kv_heads, head_dim, max_pos, 0, nullptr));
    check(flexllm_mha_i8_prefill(q8.get(), kc.get(), vc.get(), &sc, dout.get(), nullptr, seq_len, q_heads, kv_heads, head_dim, max_pos, nullptr));
    check_hip(hipEventRecord(e1, nullptr)); check_hip(hipEventSynchronize(e1));
    float ms = 0;
    check_hip(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    auto o = dout.download();
    for (int t = 0; t < seq_len; t++)
        for (int j = 0; j < H; j++) o_mmap[(size_t)(t / TP) * H + j][t % TP] = o[(size_t)t * H + j];
    return (int64_t)(ms * 1e6);
}

// MHA_i8xi8_decoding_tb (SpinQuant_Llama_32_1B/MHA_i8xi8.h:1027-1114) for ONE layer: dec_seq_len tokens are decoded one
// after another on top of pre_seq_len cached positions.  q_mmap/k_mmap/v_mmap/o_mmap use the decode packing
// [token*dim/BP + j % (dim/BP)][j / (dim/BP)] of that layer's slice; k_caches/v_caches are the reference's HP lane
// buffers in its line layouts (all layers; `layer` selects the block), read for positions < pre_seq_len and written back
// for the decoded positions, as the reference's cache managers do.  Scales: that layer's rows of Q_s/K_s/V_s/A_s.
template <int BP, int HP, int KP, int VP, int q_heads, int kv_heads, int head_dim, class VF, class VK, class VV>
void MHA_i8xi8_decoding_layer(const std::vector<VF>& q_mmap, const std::vector<VF>& k_mmap, const std::vector<VF>& v_mmap,
                              std::vector<VK>* k_caches, std::vector<VV>* v_caches, std::vector<VF>& o_mmap, const float* Q_s,
                              const float* K_s, const float* V_s, const float* A_s, int layer, int layers, int max_sum_seq_len,
                              int pre_seq_len, int dec_seq_len, float sqrt_head_dim) {
    const int H = q_heads * head_dim, KV = kv_heads * head_dim;
    const CacheGeom geom{layers, kv_heads, head_dim, max_sum_seq_len};
    const int max_pos = (pre_seq_len + dec_seq_len + 63) / 64 * 64;
    auto unpack = [&](const std::vector<VF>& mm, int dim, int t) {
        std::vector<float> x(dim);
        const int per = dim / BP;
        for (int j = 0; j < dim; j++) x[j] = mm[(size_t)t * per + j % per][j / per];
        return x;
    };
    // the cached history -> token-major -> the GPU's cache layout
    std::vector<int8_t> k_hist((size_t)pre_seq_len * KV), v_hist((size_t)pre_seq_len * KV);
    kcache_decode_to_token_major<HP, KP>(k_caches, geom, layer, pre_seq_len, k_hist.data());
    vcache_decode_to_token_major<HP, VP>(v_caches, geom, layer, pre_seq_len, v_hist.data());
    DeviceArray<int8_t> dkh(k_hist), dvh(v_hist), kc((size_t)kv_heads * max_pos * head_dim), vc((size_t)kv_heads * max_pos * head_dim);
    check_hip(hipMemset(kc.get(), 0, kc.size()));
    check_hip(hipMemset(vc.get(), 0, vc.size()));
    if (pre_seq_len > 0) check(flexllm_kv_store_i8(dkh.get(), dvh.get(), kc.get(), vc.get(), pre_seq_len, kv_heads, head_dim, max_pos, 0, nullptr));
    DeviceArray<float> dqs(std::vector<float>(Q_s, Q_s + q_heads)), dks(std::vector<float>(K_s, K_s + kv_heads)),
        dvs(std::vector<float>(V_s, V_s + kv_heads)), das(std::vector<float>(A_s, A_s + q_heads));
    flexllm_mha_scales sc{dqs.get(), dks.get(), dvs.get(), das.get()};
    DeviceArray<float> dq(H), dk(KV), dv(KV), dout(H);
    DeviceArray<int8_t> q8(H), k8(KV), v8(KV);
    for (int t = 0; t < dec_seq_len; t++) {
        const int pos = pre_seq_len + t;
        dq.upload(unpack(q_mmap, H, t));
        dk.upload(unpack(k_mmap, KV, pos));              // the k/v buffers hold all positions; the decoded ones follow the history
        dv.upload(unpack(v_mmap, KV, pos));
        check(flexllm_static_quant_i8(dq.get(), q8.get(), dqs.get(), sqrt_head_dim, 1, 1, q_heads, head_dim, nullptr));
        check(flexllm_static_quant_i8(dk.get(), k8.get(), dks.get(), 1.0f, 1, 1, kv_heads, head_dim, nullptr));
        check(flexllm_static_quant_i8(dv.get(), v8.get(), dvs.get(), 1.0f, 1, 1, kv_heads, head_dim, nullptr));
        check(flexllm_kv_store_i8(k8.get(), v8.get(), kc.get(), vc.get(), 1, kv_heads, head_dim, max_pos, pos, nullptr));
        check(flexllm_mha_i8_decode(q8.get(), kc.get(), vc.get(), &sc, dout.get(), nullptr, pos + 1, q_heads, kv_heads, head_dim, max_pos, nullptr));
        const auto k_new = k8.download(), v_new = v8.download();
        kcache_decode_from_token_major<HP, KP>(k_new.data(), geom, layer, pos, 1, k_caches);
        vcache_decode_from_token_major<HP, VP>(v_new.data(), geom, layer, pos, 1, v_caches);
        const auto o = dout.download();
        const int per = H / BP;
        for (int j = 0; j < H; j++) o_mmap[(size_t)t * per + j % per][j / per] = o[j];
    }
}

// ======================================================================================= Linear_Layer_test.h tops
// QuantWrapper_Linear_Layer_q_Decoding_tb (SpinQuant_Llama_32_1B/Linear_Layer_test.h:332-364) for ONE layer, with the
// testbench's own buffers: input_mmap / output_mmap in the decode packing [t*dim/BP + j % (dim/BP)][j / (dim/BP)],
// quant_weight_mmaps = the BP lane buffers of packed int4 weight words exactly as Linear_Layer_Decoding_tb.cpp:176-186
// fills them, weight_s_sum_mmap[n] = {scale, row sum of the dequantised weights}.  Per token: asymmetric uint4
// quantisation, int4 GEMV, dequantisation with zero point x row sum.
template <int BP, int WP, int input_dim, int output_dim, class VF, class VW, class VS>
void QuantWrapper_Linear_Layer_q_Decoding_layer(const std::vector<VF>& input_mmap, std::vector<VW>* quant_weight_mmaps,
                                                const std::vector<VS>& weight_s_sum_mmap, std::vector<VF>& output_mmap,
                                                int dec_seq_len) {
    std::vector<int8_t> row_major((size_t)output_dim * input_dim);
    unpack_weight_int4_decode<WP, BP>(quant_weight_mmaps, output_dim, input_dim, row_major.data());
    DeviceWeight4 weight(row_major.data(), output_dim, input_dim);
    std::vector<float> ws(output_dim), wsum(output_dim);
    for (int n = 0; n < output_dim; n++) { ws[n] = weight_s_sum_mmap[n][0]; wsum[n] = weight_s_sum_mmap[n][1]; }
    DeviceArray<float> dws(ws), dwsum(wsum), dx(input_dim), ds(1), db(1), dy(output_dim);
    DeviceArray<uint8_t> dq(input_dim), dq4(input_dim / 2);
    const int per_in = input_dim / BP, per_out = output_dim / BP;
    std::vector<float> x(input_dim);
    for (int t = 0; t < dec_seq_len; t++) {
        for (int j = 0; j < input_dim; j++) x[j] = input_mmap[(size_t)t * per_in + j % per_in][j / per_in];
        dx.upload(x);
        check(flexllm_quant_asym_u8(dx.get(), dq.get(), ds.get(), db.get(), 4, 1, input_dim, nullptr));
        check(flexllm_pack_nibbles(dq.get(), dq4.get(), (size_t)input_dim, nullptr));
        check(flexllm_linear_u4i4_gemv_dequant(dq4.get(), ds.get(), db.get(), weight.w4.get(), dws.get(), dwsum.get(), nullptr,
                                               dy.get(), input_dim, output_dim, nullptr));
        const auto y = dy.download();
        for (int j = 0; j < output_dim; j++) output_mmap[(size_t)t * per_out + j % per_out][j / per_out] = y[j];
    }
}
// QuantWrapper_Linear_Layer_q_Prefilling_tb (Linear_Layer_test.h:145-175) for ONE layer: input_mmap / output_mmap in the
// prefill packing [(t/TP)*dim + j][t % TP], quant_weight_mmap the packed words of Linear_Layer_Prefilling_tb.cpp:
// 226-231 (WP output channels per word group, the vector may be wider than WP/2 bytes: the read-parallel padding).
template <int TP, int WP, int input_dim, int output_dim, class VF, class VW, class VS>
void QuantWrapper_Linear_Layer_q_Prefilling_layer(const std::vector<VF>& input_mmap, const std::vector<VW>& quant_weight_mmap,
                                                  const std::vector<VS>& weight_s_sum_mmap, std::vector<VF>& output_mmap, int seq_len) {
    std::vector<int8_t> row_major((size_t)output_dim * input_dim);
    unpack_weight_int4_prefill<WP>(quant_weight_mmap, output_dim, input_dim, row_major.data());
    DeviceWeight4 weight(row_major.data(), output_dim, input_dim);
    std::vector<float> ws(output_dim), wsum(output_dim), x((size_t)seq_len * input_dim);
    for (int n = 0; n < output_dim; n++) { ws[n] = weight_s_sum_mmap[n][0]; wsum[n] = weight_s_sum_mmap[n][1]; }
    for (int t = 0; t < seq_len; t++)
        for (int j = 0; j < input_dim; j++) x[(size_t)t * input_dim + j] = input_mmap[(size_t)(t / TP) * input_dim + j][t % TP];
    DeviceArray<float> dx(x), dws(ws), dwsum(wsum), ds(seq_len), db(seq_len), dy((size_t)seq_len * output_dim);
    DeviceArray<uint8_t> dq(x.size()), dq4(x.size() / 2);
    check(flexllm_quant_asym_u8(dx.get(), dq.get(), ds.get(), db.get(), 4, seq_len, input_dim, nullptr));
    check(flexllm_pack_nibbles(dq.get(), dq4.get(), x.size(), nullptr));
    check(flexllm_linear_u4i4_gemm_dequant(dq4.get(), ds.get(), db.get(), weight.w4.get(), dws.get(), dwsum.get(), nullptr, dy.get(),
                                           seq_len, input_dim, output_dim, nullptr));
    const auto y = dy.download();
    for (int t = 0; t < seq_len; t++)
        for (int j = 0; j < output_dim; j++) output_mmap[(size_t)(t / TP) * output_dim + j][t % TP] = y[(size_t)t * output_dim + j];
}

// ======================================================================================= Logits.h
// The logits stream is block-partitioned like every decode stream: lane i of read m carries logit
// i*(logits_num/block_parallel_samp) + m (Modules/Logits.h:98).
// Modules/Logits.h:34-40: the top_k largest logits in descending order (strict '>' on insertion, so an equal value
// queues behind the one found first), softmax over them, top_k packs {index, probability}.
template <typename T, int block_parallel_samp, int max_logits_num, int top_k, int max_hidden_dim = 2048, int block_logits_num = 2048,
          int inner_block_parallel = 1, bool enable_softmax = true, bool enable_sub_max = true, class IS, class OS>
void dec_Logits_Max_K_Layer(IS& logits_stream, OS& max_logits_stream, int logits_num = max_logits_num) {
    static_assert(std::is_same<T, float>::value && enable_softmax, "fp32 logits, probabilities on the output");
    auto logits = drain_dec<float>(logits_stream, logits_num, block_parallel_samp);
    DeviceArray<float> dl(logits), dr(std::vector<float>{0.0f}), dval(top_k), dprob(top_k);
    DeviceArray<int> dtok(1), didx(top_k);
    check(flexllm_sample_topk_f32(dl.get(), logits_num, top_k, dr.get(), enable_sub_max ? 1 : 0, dtok.get(), didx.get(), dval.get(),
                                  dprob.get(), nullptr));
    const auto idx = didx.download();
    const auto prob = dprob.download();
    for (int k = 0; k < top_k; k++) {
        typename OS::value_type out_pack;
        out_pack[0] = (T)idx[k];
        out_pack[1] = prob[k];
        max_logits_stream.write(out_pack);
    }
}
// Modules/Logits.h:145-155: top-k selection and softmax as above, a draw with the host-supplied uniform number rand_seed
// (the smallest k with rand_seed < cdf[k], else the last), and the sampled token's embedding row read from vocab_lib
// (fp32 rows in the decode packing, row t at vocab_lib[t*dim/BPE ...], Modules/data_io.h:348-363) onto the stream.
template <typename T, int block_parallel_samp, int max_logits_num, int top_k, int block_parallel_embed, int max_hidden_dim = 2048,
          int block_logits_num = 2048, int inner_block_parallel = 1, bool enable_sub_max = true, class IS, class VE, class OS>
void dec_Sampling_Embedding_Layer(IS& logits_stream, const std::vector<VE>& vocab_lib, OS& new_embedding_stream, T rand_seed,
                                  int& sampled_idx, int logits_num = max_logits_num, int io_hidden_dim = max_hidden_dim) {
    static_assert(std::is_same<T, float>::value, "fp32 logits");
    auto logits = drain_dec<float>(logits_stream, logits_num, block_parallel_samp);
    DeviceArray<float> dl(logits), dr(std::vector<float>{(float)rand_seed});
    DeviceArray<int> dtok(1);
    check(flexllm_sample_topk_f32(dl.get(), logits_num, top_k, dr.get(), enable_sub_max ? 1 : 0, dtok.get(), nullptr, nullptr, nullptr, nullptr));
    sampled_idx = dtok.download()[0];
    const size_t per = (size_t)io_hidden_dim / block_parallel_embed;
    for (size_t i = 0; i < per; i++) new_embedding_stream.write(vocab_lib[(size_t)sampled_idx * per + i]);
}

}  // namespace fxhost
