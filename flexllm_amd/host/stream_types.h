// Minimal host-side carriers for harnesses that do not have TAPA / Vitis HLS at hand: a FIFO with the
// read()/write() surface of tapa::istream / tapa::ostream and a fixed-size vector with the operator[] surface
// of hls::vector.  The module functions in flexllm_modules.h are templates over the stream type, so code that
// does have TAPA passes tapa::stream<hls::vector<T,N>> instead and nothing here is needed.
#pragma once
#include <cstddef>
#include <deque>
#include <stdexcept>

namespace fxhost {

template <class T, int N>
struct vec {
    using value_type = T;
    static constexpr int size = N;
    T v[N];
    T& operator[](int i) { return v[i]; }
    const T& operator[](int i) const { return v[i]; }
};

// Unbounded FIFO.  The GPU-backed modules consume their whole input before producing output, so harness code
// calls them one after another on a single thread (no task graph is needed for correctness).
template <class V>
class stream {
public:
    using value_type = V;
    void write(const V& x) { q_.push_back(x); }
    V read() {
        if (q_.empty()) throw std::runtime_error("fxhost::stream: read from an empty stream");
        V x = q_.front();
        q_.pop_front();
        return x;
    }
    bool empty() const { return q_.empty(); }
    size_t size() const { return q_.size(); }

private:
    std::deque<V> q_;
};

}  // namespace fxhost
