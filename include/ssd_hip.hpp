// C++ host side of libssd_hip: what the reference's Rust host side would be, written in the one compiled host
// language this build has.  It mirrors the shape of the reference's op wrappers -- validate the tensors, call the
// extern "C" entry point with raw device pointers, turn a non-zero return code into an error carrying the
// library's thread-local message (trading_bots/src/torch/fa4.rs:145-191 for the validate-then-call shape,
// trading_bots/src/torch/cuda/graph.rs:107-119 for fetching and freeing the message) -- and the life cycle of
// the reference's recurrent memory (trading_bots/src/torch/model/trading_model.rs:56-75 StreamState;
// trading_bots/src/torch/model/stream/state.rs:10-21 reset, :52-110 build; per-env reset
// trading_bots/src/torch/train/rollout.rs:130-135).
//
// Ownership follows the reference: tensors stay with the caller, the wrappers allocate only their outputs and
// the workspace, and owning types release in their destructors (the RAII handles of graph.rs:8-11,100-105).
// Header-only; link with libssd_hip.so and the HIP runtime.
#pragma once
#include <hip/hip_runtime.h>

#include <array>
#include <cstdint>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <utility>

#include "ssd_hip.h"

namespace ssd_hip {

// A failed call: the library's return code and message (anyhow::Error in the reference's wrappers).
class Error : public std::runtime_error {
public:
    Error(int code, const std::string &what) : std::runtime_error(what), code_(code) {}
    int code() const { return code_; }

private:
    int code_;
};

inline void check(int rc) {
    if (rc == SSD_OK) return;
    char *msg = ssd_get_and_reset_last_err();
    std::string text = msg ? msg : "unknown";
    std::free(msg);
    throw Error(rc, "ssd error " + std::to_string(rc) + ": " + text);
}

inline void check_hip(hipError_t e, const char *what) {
    if (e != hipSuccess) throw Error(SSD_ERR_RUNTIME, std::string(what) + ": " + hipGetErrorString(e));
}

enum class DType { F32 = SSD_DTYPE_F32, BF16 = SSD_DTYPE_BF16 };
inline size_t element_size(DType t) { return t == DType::F32 ? 4 : 2; }

// Device memory owned by this object (the part of a tch Tensor these wrappers need).
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t bytes) : bytes_(bytes) {
        if (bytes) check_hip(hipMalloc(&ptr_, bytes), "hipMalloc");
    }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        if (this != &o) {
            release();
            ptr_ = o.ptr_;
            bytes_ = o.bytes_;
            o.ptr_ = nullptr;
            o.bytes_ = 0;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }
    void *data() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    void upload(const void *host, size_t n) { check_hip(hipMemcpy(ptr_, host, n, hipMemcpyHostToDevice), "hipMemcpy H2D"); }
    void download(void *host, size_t n) const { check_hip(hipMemcpy(host, ptr_, n, hipMemcpyDeviceToHost), "hipMemcpy D2H"); }
    void zero(hipStream_t st = nullptr) { if (bytes_) check_hip(hipMemsetAsync(ptr_, 0, bytes_, st), "hipMemsetAsync"); }

private:
    void release() {
        if (ptr_) (void)hipFree(ptr_);
        ptr_ = nullptr;
    }
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

// A contiguous row-major device tensor that somebody else owns: pointer, element type, shape.
struct TensorView {
    const void *ptr = nullptr;
    DType dtype = DType::F32;
    std::array<int64_t, 4> shape{{0, 0, 0, 0}};
    int rank = 0;
    int64_t numel() const {
        int64_t n = 1;
        for (int i = 0; i < rank; ++i) n *= shape[i];
        return n;
    }
};

inline TensorView view(const void *ptr, DType t, std::initializer_list<int64_t> shape) {
    TensorView v;
    v.ptr = ptr;
    v.dtype = t;
    v.rank = (int)shape.size();
    if (v.rank > 4) throw Error(SSD_ERR_INVALID, "ssd: tensors have at most 4 dimensions");
    int i = 0;
    for (int64_t s : shape) v.shape[i++] = s;
    return v;
}

namespace detail {
inline void require(const TensorView &t, const char *name, DType dtype, std::initializer_list<int64_t> shape) {
    bool ok = t.ptr != nullptr && t.rank == (int)shape.size() && t.dtype == dtype;
    int i = 0;
    for (int64_t s : shape) ok = ok && t.shape[i++] == s;
    if (!ok) {
        std::string want;
        for (int64_t s : shape) want += (want.empty() ? "[" : ",") + std::to_string(s);
        throw Error(SSD_ERR_INVALID, std::string("SSD ") + name + " must be a " + (dtype == DType::F32 ? "float32" : "bfloat16") +
                                         " tensor of shape " + want + "]");
    }
}
}  // namespace detail

// Outputs of the forward: y [B,L,H,P] in x's type and the final state [B,H,P,N] float32.
struct ScanOutput {
    DeviceBuffer y, final_states;
};

// y, final = ssd_chunk_scan(x, dt, A, B, C, D, chunk, initial_states): the signature the model code would call
// (x [B,L,H,P], dt [B,L,H], A [H] f32, B, C [B,L,G,N], D [H] f32 or none, initial_states [B,H,P,N] f32 or none).
inline ScanOutput ssd_chunk_scan(const TensorView &x, const TensorView &dt, const TensorView &A, const TensorView &Bm,
                                 const TensorView &Cm, const TensorView *D, int64_t chunk, const TensorView *initial_states,
                                 hipStream_t stream = nullptr) {
    if (x.rank != 4 || Bm.rank != 4) throw Error(SSD_ERR_INVALID, "SSD x must be [B,L,H,P] and B [B,L,G,N]");
    const int64_t B = x.shape[0], L = x.shape[1], H = x.shape[2], P = x.shape[3], G = Bm.shape[2], N = Bm.shape[3];
    detail::require(dt, "dt", x.dtype, {B, L, H});
    detail::require(A, "A", DType::F32, {H});
    detail::require(Bm, "B", x.dtype, {B, L, G, N});
    detail::require(Cm, "C", x.dtype, {B, L, G, N});
    if (D) detail::require(*D, "D", DType::F32, {H});
    if (initial_states) detail::require(*initial_states, "initial_states", DType::F32, {B, H, P, N});
    const ssd_dims dims = {B, L, H, P, N, G, chunk};
    size_t need = 0;
    check(ssd_workspace_bytes(&dims, &need));
    DeviceBuffer ws(need);
    ScanOutput out{DeviceBuffer((size_t)x.numel() * element_size(x.dtype)), DeviceBuffer((size_t)(B * H * P * N) * 4)};
    check(ssd_chunk_scan_fwd(&dims, (int)x.dtype, x.ptr, dt.ptr, static_cast<const float *>(A.ptr), Bm.ptr, Cm.ptr,
                             D ? static_cast<const float *>(D->ptr) : nullptr,
                             initial_states ? static_cast<const float *>(initial_states->ptr) : nullptr, out.y.data(),
                             static_cast<float *>(out.final_states.data()), ws.data(), need, stream));
    // the workspace is released when this returns: wait for the kernels that use it
    check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return out;
}

// The recurrent memory of the streams: [B,H,P,N] float32, zero at the start; rows are zeroed per environment.
class StreamState {
public:
    StreamState(int64_t batch, int64_t nheads, int64_t headdim, int64_t dstate)
        : B_(batch), H_(nheads), P_(headdim), N_(dstate), buf_((size_t)(batch * nheads * headdim * dstate) * 4) {
        reset();
    }
    // all streams back to the empty state (stream/state.rs:10-21)
    void reset(hipStream_t st = nullptr) { buf_.zero(st); }
    // one environment's stream back to the empty state (train/rollout.rs:130-135)
    void reset_row(int64_t row, hipStream_t st = nullptr) {
        if (row < 0 || row >= B_) throw Error(SSD_ERR_INVALID, "SSD stream row out of range");
        const size_t per = (size_t)(H_ * P_ * N_) * 4;
        check_hip(hipMemsetAsync(static_cast<char *>(buf_.data()) + row * per, 0, per, st), "hipMemsetAsync");
    }
    // continue the streams from the end of a scanned prefix: its final state becomes the memory
    void adopt(const DeviceBuffer &final_states, hipStream_t st = nullptr) {
        if (final_states.bytes() != buf_.bytes()) throw Error(SSD_ERR_INVALID, "SSD final state has another size");
        check_hip(hipMemcpyAsync(buf_.data(), final_states.data(), buf_.bytes(), hipMemcpyDeviceToDevice, st), "hipMemcpyAsync");
    }
    float *data() const { return static_cast<float *>(buf_.data()); }
    TensorView as_view() const { return view(buf_.data(), DType::F32, {B_, H_, P_, N_}); }
    int64_t batch() const { return B_; }
    int64_t nheads() const { return H_; }
    int64_t headdim() const { return P_; }
    int64_t dstate() const { return N_; }

private:
    int64_t B_, H_, P_, N_;
    DeviceBuffer buf_;
};

// y = ssd_step(state, x, dt, A, B, C, D): advances every stream by one timestep in place
// (x [B,H,P], dt [B,H], B, C [B,G,N]); returns y [B,H,P] in x's type.
inline DeviceBuffer ssd_step(StreamState &state, const TensorView &x, const TensorView &dt, const TensorView &A,
                             const TensorView &Bm, const TensorView &Cm, const TensorView *D, hipStream_t stream = nullptr) {
    if (Bm.rank != 3) throw Error(SSD_ERR_INVALID, "SSD step B must be [B,G,N]");
    const int64_t B = state.batch(), H = state.nheads(), P = state.headdim(), N = state.dstate(), G = Bm.shape[1];
    detail::require(x, "x", x.dtype, {B, H, P});
    detail::require(dt, "dt", x.dtype, {B, H});
    detail::require(A, "A", DType::F32, {H});
    detail::require(Bm, "B", x.dtype, {B, G, N});
    detail::require(Cm, "C", x.dtype, {B, G, N});
    if (D) detail::require(*D, "D", DType::F32, {H});
    const ssd_step_dims dims = {B, H, P, N, G};
    DeviceBuffer y((size_t)x.numel() * element_size(x.dtype));
    check(ssd_step_fwd(&dims, (int)x.dtype, state.data(), x.ptr, dt.ptr, static_cast<const float *>(A.ptr), Bm.ptr, Cm.ptr,
                       D ? static_cast<const float *>(D->ptr) : nullptr, y.data(), stream));
    return y;
}

// y = ssd_steps(state, x, dt, A, B, C, D, reset): advances every stream by T timesteps in one call, in place
// (x [B,T,H,P], dt [B,T,H], B, C [B,T,G,N]: the scan's layout; reset: device pointer to [B,T] bytes or NULL, a
// non-zero byte empties that stream right before the step -- the rollout's advance -> reset slots -> forward,
// train/rollout.rs:130-135,209-235); returns y [B,T,H,P] in x's type.
inline DeviceBuffer ssd_steps(StreamState &state, const TensorView &x, const TensorView &dt, const TensorView &A,
                              const TensorView &Bm, const TensorView &Cm, const TensorView *D,
                              const uint8_t *reset = nullptr, hipStream_t stream = nullptr) {
    if (x.rank != 4 || Bm.rank != 4) throw Error(SSD_ERR_INVALID, "SSD steps x must be [B,T,H,P] and B [B,T,G,N]");
    const int64_t B = state.batch(), H = state.nheads(), P = state.headdim(), N = state.dstate(), T = x.shape[1],
                  G = Bm.shape[2];
    detail::require(x, "x", x.dtype, {B, T, H, P});
    detail::require(dt, "dt", x.dtype, {B, T, H});
    detail::require(A, "A", DType::F32, {H});
    detail::require(Bm, "B", x.dtype, {B, T, G, N});
    detail::require(Cm, "C", x.dtype, {B, T, G, N});
    if (D) detail::require(*D, "D", DType::F32, {H});
    const ssd_step_dims dims = {B, H, P, N, G};
    DeviceBuffer y((size_t)x.numel() * element_size(x.dtype));
    check(ssd_steps_fwd(&dims, T, (int)x.dtype, state.data(), reset, x.ptr, dt.ptr, static_cast<const float *>(A.ptr), Bm.ptr,
                        Cm.ptr, D ? static_cast<const float *>(D->ptr) : nullptr, y.data(), stream));
    return y;
}

}  // namespace ssd_hip
