// HIP backend of the host mirror.  Keeps the parts of include/motifcl/runtime/backend.hpp:14-86
// the counter layer uses: a lifetime handle, create(), finish(), device_info(); the single
// in-order queue of the reference is one HIP stream.
#pragma once

#include <memory>
#include <string>

namespace motifcl {

struct BackendLifetime {
    bool alive = true;
};

enum class BackendKind { Hip };

struct DeviceInfo {
    std::string name;
};

class Backend {
public:
    Backend() = default;
    ~Backend();

    Backend(const Backend&) = delete;
    Backend& operator=(const Backend&) = delete;
    Backend(Backend&& other) noexcept;
    Backend& operator=(Backend&& other) noexcept;

    static Backend create_hip();
    static Backend create() { return create_hip(); }

    BackendKind kind() const { return BackendKind::Hip; }
    bool is_hip() const { return true; }
    bool is_vulkan() const { return false; }
    bool is_opencl() const { return false; }
    void* hip_stream() const { return stream_; }  // hipStream_t; nullptr is the default stream

    void finish() const;
    DeviceInfo device_info() const;
    std::shared_ptr<BackendLifetime> lifetime_handle() const { return lifetime_; }

    // Transient workspace shared by every layer of this backend (the fused update's gradient
    // strip); grows to the largest request and is returned to the pool with the backend.
    void* workspace(std::size_t nbytes);
    std::size_t workspace_nbytes() const { return workspace_nbytes_; }
    void release_workspace();

private:
    void* stream_ = nullptr;
    void* workspace_ = nullptr;
    std::size_t workspace_nbytes_ = 0;
    std::shared_ptr<BackendLifetime> lifetime_ = std::make_shared<BackendLifetime>();
};

// Device-memory accounting (src/runtime/buffer.cpp:28-33 of MotifCL).
std::size_t device_bytes_current();
std::size_t device_bytes_peak();
void device_bytes_reset_peak();

}  // namespace motifcl
