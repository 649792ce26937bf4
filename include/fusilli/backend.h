// Backend, Handle and Buffer: device, stream and memory ownership for the
// graph API, implemented on the C ABI of fusilli_hip.h.
//
// Same surface and error behaviour as the reference (backend/backend.h:42-57,
// backend/handle.h:35-176, backend/buffer.h:31-81, backend/runtime.h:531-674)
// with the IREE types removed: a Handle is a device + stream context, a Buffer
// is a device allocation (or a non-owning view of caller memory).
// Backend::AMDGPU executes; Backend::CPU exists so that graphs can be built,
// validated, planned and serialised on a machine without a GPU — it holds
// host memory and has no execution engine.
#ifndef FUSILLI_BACKEND_H
#define FUSILLI_BACKEND_H

#include <cstring>
#include <memory>
#include <ostream>
#include <string>
#include <vector>

#include "../fusilli_hip.h"
#include "errors.h"
#include "types.h"

namespace fusilli {

enum class Backend : uint8_t { CPU, AMDGPU };

inline const char *backendName(Backend b) {
  return b == Backend::CPU ? "CPU" : b == Backend::AMDGPU ? "AMDGPU"
                                                          : "UNKNOWN_BACKEND";
}
inline std::ostream &operator<<(std::ostream &os, const Backend &b) {
  return os << backendName(b);
}
// Whether execute() returns before the device has finished.
inline bool backendExecutesAsync(Backend b) { return b == Backend::AMDGPU; }

class Buffer;
class Graph;

class Handle {
public:
  // Device 0, a stream owned by the handle.
  static ErrorOr<Handle> create(Backend backend) {
    if (backend == Backend::CPU)
      return ok(Handle(backend, nullptr));
    if (backend != Backend::AMDGPU)
      return error(ErrorCode::InternalError,
                   "Handle::create got an unknown backend");
    return createAmdgpu(/*deviceId=*/0, /*stream=*/0);
  }
  static ErrorOr<Handle> create(Backend backend, int deviceId) {
    return create(backend, deviceId, 0);
  }
  // `stream` is a hipStream_t the caller owns (0 = create one).
  static ErrorOr<Handle> create(Backend backend, int deviceId,
                                uintptr_t stream) {
    FUSILLI_RETURN_ERROR_IF(backend != Backend::AMDGPU,
                            ErrorCode::InvalidArgument,
                            "Stream can only be set on AMDGPU backend");
    return createAmdgpu(deviceId, stream);
  }

  Handle(const Handle &) = delete;
  Handle &operator=(const Handle &) = delete;
  Handle(Handle &&) noexcept = default;
  Handle &operator=(Handle &&) noexcept = default;
  ~Handle() = default;

  Backend getBackend() const { return backend_; }
  // The C-ABI context (null for Backend::CPU).
  fhip_ctx *getContext() const { return ctx_.get(); }
  // Shared ownership of the context, for objects that must outlive the handle.
  const std::shared_ptr<fhip_ctx> &getSharedContext() const { return ctx_; }
  // Blocks until everything queued on the handle's stream has finished.
  ErrorObject synchronize() const {
    if (!ctx_)
      return ok();
    FUSILLI_RETURN_ERROR_IF(fhip_stream_sync(ctx_.get()) != 0,
                            ErrorCode::RuntimeFailure,
                            std::string(fhip_last_error(ctx_.get())));
    return ok();
  }

private:
  Handle(Backend b, fhip_ctx *c)
      : backend_(b),
        ctx_(c, [](fhip_ctx *p) {
          if (p)
            fhip_ctx_destroy(p);
        }) {}

  static ErrorOr<Handle> createAmdgpu(int deviceId, uintptr_t stream) {
    fhip_ctx *ctx = nullptr;
    const int rc =
        fhip_ctx_create(deviceId, reinterpret_cast<void *>(stream), &ctx);
    FUSILLI_RETURN_ERROR_IF(rc != 0, ErrorCode::RuntimeFailure,
                            std::string(fhip_last_error(nullptr)));
    return ok(Handle(Backend::AMDGPU, ctx));
  }

  Backend backend_;
  std::shared_ptr<fhip_ctx> ctx_;
};

// A device buffer (AMDGPU) or host buffer (CPU handle).  Move-only.
class Buffer {
public:
  // New buffer of shape `bufferShape` filled with `bufferData`
  // (backend/runtime.h:531-582).
  template <typename T>
  static ErrorOr<Buffer> allocate(const Handle &handle,
                                  const std::vector<size_t> &bufferShape,
                                  const std::vector<T> &bufferData) {
    size_t expected = 1;
    for (size_t d : bufferShape)
      expected *= d;
    FUSILLI_RETURN_ERROR_IF(
        expected == 0 || bufferShape.empty(), ErrorCode::RuntimeFailure,
        "Buffer::allocate failed: cannot allocate a buffer with zero size");
    FUSILLI_RETURN_ERROR_IF(
        bufferData.size() != expected, ErrorCode::RuntimeFailure,
        "Buffer::allocate failed: bufferData size (" +
            std::to_string(bufferData.size()) +
            ") does not match product of bufferShape dimensions (" +
            std::to_string(expected) + ")");
    FUSILLI_ASSIGN_OR_RETURN(Buffer buf,
                             allocateRaw(handle, expected * sizeof(T)));
    buf.dataType_ = DataTypeOf<T>::value;
    buf.shape_ = bufferShape;
    buf.typed_ = true;
    if constexpr (std::is_same_v<T, bool>) {
      std::vector<uint8_t> bytes(bufferData.begin(), bufferData.end());
      FUSILLI_CHECK_ERROR(buf.upload(handle, bytes.data(), bytes.size()));
    } else {
      FUSILLI_CHECK_ERROR(
          buf.upload(handle, bufferData.data(), expected * sizeof(T)));
    }
    return ok(std::move(buf));
  }

  // Non-owning view of device memory the caller allocated (hipMalloc or
  // hipMallocAsync); the caller keeps it alive while the Buffer is in use.
  // Replaces the reference's import of an IREE buffer view
  // (backend/runtime.h:584-593).
  static ErrorOr<Buffer> import(void *devicePtr, size_t sizeInBytes,
                                DataType dataType = DataType::NotSet) {
    FUSILLI_RETURN_ERROR_IF(devicePtr == nullptr, ErrorCode::RuntimeFailure,
                            "Buffer::import failed as the external pointer "
                            "is NULL");
    Buffer b;
    b.ptr_ = devicePtr;
    b.bytes_ = sizeInBytes;
    b.dataType_ = dataType;
    b.typed_ = dataType != DataType::NotSet;
    b.owned_ = false;
    b.onDevice_ = true;
    return ok(std::move(b));
  }

  // Untyped buffer, e.g. a workspace (backend/runtime.h:595-624).
  static ErrorOr<Buffer> allocateRaw(const Handle &handle, size_t sizeInBytes) {
    FUSILLI_RETURN_ERROR_IF(sizeInBytes == 0, ErrorCode::RuntimeFailure,
                            "Buffer::allocateRaw failed: cannot allocate "
                            "zero-size buffer");
    Buffer b;
    b.bytes_ = sizeInBytes;
    b.dataType_ = DataType::Int8;
    b.shape_ = {sizeInBytes};
    b.owned_ = true;
    if (handle.getBackend() == Backend::AMDGPU) {
      b.ctx_ = handle.getSharedContext();
      b.onDevice_ = true;
      FUSILLI_RETURN_ERROR_IF(
          fhip_malloc(b.ctx_.get(), sizeInBytes, &b.ptr_) != 0,
          ErrorCode::RuntimeFailure,
          std::string(fhip_last_error(b.ctx_.get())));
    } else {
      b.onDevice_ = false;
      b.ptr_ = std::malloc(sizeInBytes);
      FUSILLI_RETURN_ERROR_IF(b.ptr_ == nullptr, ErrorCode::RuntimeFailure,
                              "Buffer::allocateRaw failed: out of host memory");
    }
    return ok(std::move(b));
  }

  // Copies the whole buffer to `outData` (which must be empty); waits for all
  // work queued on the handle's stream first (backend/runtime.h:646-674).
  template <typename T>
  ErrorObject read(const Handle &handle, std::vector<T> &outData) {
    FUSILLI_RETURN_ERROR_IF(outData.size() != 0, ErrorCode::RuntimeFailure,
                            "Buffer::read failed as outData is NOT empty");
    FUSILLI_RETURN_ERROR_IF(ptr_ == nullptr, ErrorCode::RuntimeFailure,
                            "Buffer::read failed as the buffer is empty");
    if constexpr (std::is_same_v<T, bool>) {
      std::vector<uint8_t> bytes(bytes_);
      FUSILLI_CHECK_ERROR(download(handle, bytes.data(), bytes_));
      outData.assign(bytes.begin(), bytes.end());
    } else {
      outData.resize(bytes_ / sizeof(T));
      FUSILLI_CHECK_ERROR(download(handle, outData.data(),
                                   outData.size() * sizeof(T)));
    }
    return ok();
  }

  Buffer(const Buffer &) = delete;
  Buffer &operator=(const Buffer &) = delete;
  Buffer(Buffer &&o) noexcept { steal(o); }
  Buffer &operator=(Buffer &&o) noexcept {
    if (this != &o) {
      release();
      steal(o);
    }
    return *this;
  }
  ~Buffer() { release(); }

  void *data() const { return ptr_; }
  size_t sizeInBytes() const { return bytes_; }
  DataType getDataType() const { return dataType_; }
  const std::vector<size_t> &getShape() const { return shape_; }
  bool isDeviceMemory() const { return onDevice_; }
  // True when the element type was given (allocate<T>, typed import).
  bool isTyped() const { return typed_; }
  explicit operator bool() const { return ptr_ != nullptr; }
  bool operator==(std::nullptr_t) const { return ptr_ == nullptr; }
  bool operator!=(std::nullptr_t) const { return ptr_ != nullptr; }

private:
  Buffer() = default;

  ErrorObject upload(const Handle &handle, const void *src, size_t n) {
    if (onDevice_) {
      FUSILLI_RETURN_ERROR_IF(fhip_memcpy_h2d(handle.getContext(), ptr_, src,
                                              n) != 0,
                              ErrorCode::RuntimeFailure,
                              std::string(fhip_last_error(handle.getContext())));
    } else {
      std::memcpy(ptr_, src, n);
    }
    return ok();
  }
  ErrorObject download(const Handle &handle, void *dst, size_t n) const {
    if (onDevice_) {
      FUSILLI_RETURN_ERROR_IF(
          handle.getBackend() != Backend::AMDGPU, ErrorCode::InvalidArgument,
          "Buffer::read needs the AMDGPU handle the buffer lives on");
      FUSILLI_RETURN_ERROR_IF(fhip_memcpy_d2h(handle.getContext(), dst, ptr_,
                                              n) != 0,
                              ErrorCode::RuntimeFailure,
                              std::string(fhip_last_error(handle.getContext())));
    } else {
      std::memcpy(dst, ptr_, n);
    }
    return ok();
  }
  void release() {
    if (ptr_ && owned_) {
      if (onDevice_)
        fhip_free(ctx_.get(), ptr_);
      else
        std::free(ptr_);
    }
    ptr_ = nullptr;
  }
  void steal(Buffer &o) {
    ptr_ = o.ptr_;
    bytes_ = o.bytes_;
    dataType_ = o.dataType_;
    shape_ = std::move(o.shape_);
    owned_ = o.owned_;
    onDevice_ = o.onDevice_;
    typed_ = o.typed_;
    ctx_ = std::move(o.ctx_);
    o.ptr_ = nullptr;
    o.bytes_ = 0;
  }

  void *ptr_ = nullptr;
  size_t bytes_ = 0;
  DataType dataType_ = DataType::NotSet;
  std::vector<size_t> shape_;
  bool owned_ = false;
  bool onDevice_ = false;
  bool typed_ = false;
  std::shared_ptr<fhip_ctx> ctx_; // keeps the allocating context alive
};

} // namespace fusilli

#endif // FUSILLI_BACKEND_H
