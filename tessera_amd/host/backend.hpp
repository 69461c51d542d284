// C++20 host side of the MI355X quantized-matmul backend: the reference's `Backend`
// interface (include/tessera/backend.hpp:45-134,847-1037) restated over the C ABI of
// libtessera_qmm.so, with the same method names, argument meaning and error behaviour, so
// that code written against the reference reads the same here.  The reference returns
// std::expected<T, StatusCode> (C++23); this header carries a small Expected<T> with the same
// surface (has_value / operator bool / operator* / value / error) because the toolchain this
// library is built with stops at C++20.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <memory>
#include <span>
#include <string>
#include <string_view>
#include <utility>
#include <variant>
#include <vector>

#include "../../include/tessera_qmm.h"

namespace tessera_amd {

// include/tessera/types.hpp:36-48 -- same names, same integers.
enum class StatusCode : int {
  Ok = 0, InvalidArgument = 1, FileNotFound = 2, MalformedFile = 3, UnsupportedFeature = 4,
  OutOfMemory = 5, DeviceError = 6, NonFinite = 7, NetworkError = 8
};

struct Unexpected {
  StatusCode code;
};
inline Unexpected unexpected(StatusCode code) { return Unexpected{code}; }

template <class T>
class Expected {
 public:
  Expected(T value) : v_(std::move(value)) {}
  Expected(Unexpected u) : v_(u.code) {}
  bool has_value() const { return v_.index() == 0; }
  explicit operator bool() const { return has_value(); }
  T& operator*() { return std::get<0>(v_); }
  const T& operator*() const { return std::get<0>(v_); }
  T* operator->() { return &std::get<0>(v_); }
  T& value() { return std::get<0>(v_); }
  StatusCode error() const { return std::get<1>(v_); }

 private:
  std::variant<T, StatusCode> v_;
};
template <>
class Expected<void> {
 public:
  Expected() = default;
  Expected(Unexpected u) : code_(u.code) {}
  bool has_value() const { return code_ == StatusCode::Ok; }
  explicit operator bool() const { return has_value(); }
  StatusCode error() const { return code_; }

 private:
  StatusCode code_ = StatusCode::Ok;
};

enum class MemoryKind { Device };

// Weight formats of the quantized-matmul path (include/tessera/types.hpp:89-113).
enum class DType { F32, Q4K, Q5K, Q6K, F4E2M1, F8E4M3 };

class Backend;

// Move-only device allocation; frees through its backend (include/tessera/backend.hpp:69-103).
class Buffer {
 public:
  Buffer(Backend* owner, void* handle, std::size_t bytes) : owner_(owner), handle_(handle), bytes_(bytes) {}
  Buffer(const Buffer&) = delete;
  Buffer& operator=(const Buffer&) = delete;
  ~Buffer();
  void* Handle() const { return handle_; }
  std::size_t Size() const { return bytes_; }

 private:
  Backend* owner_;
  void* handle_;
  std::size_t bytes_;
};

// A loaded built-in kernel (include/tessera/backend.hpp:105-134).
class Kernel {
 public:
  Kernel(qmm_kernel handle, std::string id) : handle_(handle), id_(std::move(id)) {}
  const std::string& Id() const { return id_; }
  qmm_kernel Handle() const { return handle_; }

 private:
  qmm_kernel handle_;
  std::string id_;
};

// include/tessera/backend.hpp:45-67: buffers bind first, then each scalar as 64 bits.
struct KernelLaunch {
  std::uint32_t grid_x = 1, grid_y = 1, grid_z = 1;
  std::uint32_t block_x = 256, block_y = 1, block_z = 1;
  std::vector<const Buffer*> buffers;
  std::vector<std::uint64_t> scalars;
};

struct DeviceMemoryInfo {
  std::uint64_t total_bytes = 0, free_bytes = 0;
};

class Backend {
 public:
  std::string_view Name() const { return "mi355x"; }
  std::string_view DeviceName() const { return qmm_device_name(); }
  void SetDeviceIndex(int index) { device_ = index; }
  int DeviceIndex() const { return device_; }
  void SetStream(void* hip_stream) { stream_ = hip_stream; }

  Expected<void> Init() { return Check(qmm_init(device_)); }

  DeviceMemoryInfo MemoryInfo() const {
    DeviceMemoryInfo info;
    qmm_memory_info(&info.total_bytes, &info.free_bytes);
    return info;
  }

  Expected<std::unique_ptr<Buffer>> AllocateBuffer(std::size_t bytes, MemoryKind = MemoryKind::Device) {
    void* p = nullptr;
    if (const qmm_status rc = qmm_alloc(bytes, &p); rc != QMM_OK) return unexpected(static_cast<StatusCode>(rc));
    return std::make_unique<Buffer>(this, p, bytes);
  }
  void FreeBuffer(MemoryKind, void* handle) { qmm_free(handle); }

  Expected<void> CopyH2D(Buffer& dst, std::span<const std::byte> src) { return CopyH2DAt(dst, 0, src); }
  Expected<void> CopyH2DAt(Buffer& dst, std::size_t offset, std::span<const std::byte> src) {
    if (offset > dst.Size() || src.size() > dst.Size() - offset) return unexpected(StatusCode::InvalidArgument);
    return Check(qmm_copy_h2d(static_cast<char*>(dst.Handle()) + offset, src.data(), src.size(), stream_));
  }
  Expected<void> CopyD2H(const Buffer& src, std::span<std::byte> dst) { return CopyD2HAt(src, 0, dst); }
  Expected<void> CopyD2HAt(const Buffer& src, std::size_t offset, std::span<std::byte> dst) {
    if (offset > src.Size() || dst.size() > src.Size() - offset) return unexpected(StatusCode::InvalidArgument);
    return Check(qmm_copy_d2h(dst.data(), static_cast<const char*>(src.Handle()) + offset, dst.size(), stream_));
  }
  Expected<void> CopyD2D(const Buffer& src, std::size_t src_offset, Buffer& dst, std::size_t dst_offset,
                         std::size_t bytes) {
    if (src_offset > src.Size() || bytes > src.Size() - src_offset || dst_offset > dst.Size() ||
        bytes > dst.Size() - dst_offset) {
      return unexpected(StatusCode::InvalidArgument);
    }
    return Check(qmm_copy_d2d(static_cast<char*>(dst.Handle()) + dst_offset,
                              static_cast<const char*>(src.Handle()) + src_offset, bytes, stream_));
  }

  // Built-ins only, like RocmBackend: a non-empty `code` or an id this backend does not
  // implement is UnsupportedFeature (src/backends/rocm/rocm_backend.cpp:639-670).
  Expected<std::unique_ptr<Kernel>> LoadKernel(std::string_view name, std::span<const std::byte> code = {}) {
    if (!code.empty()) return unexpected(StatusCode::UnsupportedFeature);
    qmm_kernel k = 0;
    const std::string id(name);
    if (const qmm_status rc = qmm_load(id.c_str(), &k); rc != QMM_OK) return unexpected(static_cast<StatusCode>(rc));
    return std::make_unique<Kernel>(k, id);
  }
  void FreeKernel(void*) {}

  Expected<void> LaunchKernel(const Kernel& kernel, const KernelLaunch& launch) {
    if (launch.buffers.size() > QMM_MAX_BOUND_BUFFERS || launch.scalars.size() > QMM_MAX_SCALARS) {
      return unexpected(StatusCode::InvalidArgument);
    }
    void* bufs[QMM_MAX_BOUND_BUFFERS];
    std::size_t sizes[QMM_MAX_BOUND_BUFFERS];
    for (std::size_t i = 0; i < launch.buffers.size(); ++i) {
      if (launch.buffers[i] == nullptr) return unexpected(StatusCode::InvalidArgument);
      bufs[i] = launch.buffers[i]->Handle();
      sizes[i] = launch.buffers[i]->Size();
    }
    const std::uint32_t grid[3] = {launch.grid_x, launch.grid_y, launch.grid_z};
    const std::uint32_t block[3] = {launch.block_x, launch.block_y, launch.block_z};
    return Check(qmm_launch(kernel.Handle(), grid, block, bufs, sizes, launch.buffers.size(), launch.scalars.data(),
                            launch.scalars.size(), stream_));
  }

  void Synchronize() { qmm_sync(stream_); }
  const char* LastError() const { return qmm_last_error(); }

 private:
  static Expected<void> Check(qmm_status rc) {
    if (rc == QMM_OK) return {};
    return unexpected(static_cast<StatusCode>(rc));
  }
  int device_ = 0;
  void* stream_ = nullptr;
};

inline Buffer::~Buffer() {
  if (owner_ != nullptr && handle_ != nullptr) owner_->FreeBuffer(MemoryKind::Device, handle_);
}

// include/tessera/backend.hpp:1062-1071.
inline std::unique_ptr<Backend> CreateBackend() { return std::make_unique<Backend>(); }

}  // namespace tessera_amd
