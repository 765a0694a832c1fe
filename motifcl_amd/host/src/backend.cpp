#include <motifcl/runtime/backend.hpp>

#include <motifcl/core/error.hpp>
#include <motifcl/tensor/storage.hpp>

#include <motifcl_amd.h>

#include <utility>

namespace motifcl {

Backend Backend::create_hip() {
    Backend b;
    const std::string name = mcc_device_name();
    MCL_CHECK(!name.empty(), "no HIP device available");
    return b;  // the default stream is the backend's single in-order queue
}

Backend::~Backend() {
    if (lifetime_) lifetime_->alive = false;
    if (workspace_) mcc_device_free(workspace_);
}

Backend::Backend(Backend&& other) noexcept { *this = std::move(other); }

Backend& Backend::operator=(Backend&& other) noexcept {
    if (this != &other) {
        if (workspace_) mcc_device_free(workspace_);
        stream_ = other.stream_;
        workspace_ = other.workspace_;
        workspace_nbytes_ = other.workspace_nbytes_;
        lifetime_ = std::move(other.lifetime_);
        other.workspace_ = nullptr;
        other.workspace_nbytes_ = 0;
        other.lifetime_ = nullptr;
    }
    return *this;
}

void Backend::finish() const {
    MCL_CHECK(mcc_stream_synchronize(stream_) == MCC_OK, std::string("finish failed: ") + mcc_last_error());
}

DeviceInfo Backend::device_info() const { return DeviceInfo{mcc_device_name()}; }

void* Backend::workspace(std::size_t nbytes) {
    if (nbytes > workspace_nbytes_) {
        if (workspace_) {
            finish();  // earlier work may still read the old block
            mcc_device_free(workspace_);
            workspace_ = nullptr;
            workspace_nbytes_ = 0;
        }
        MCL_CHECK(mcc_device_alloc(&workspace_, nbytes) == MCC_OK,
                  std::string("workspace allocation failed: ") + mcc_last_error());
        workspace_nbytes_ = nbytes;
    }
    return workspace_;
}

void Backend::release_workspace() {
    if (!workspace_) return;
    finish();
    mcc_device_free(workspace_);
    workspace_ = nullptr;
    workspace_nbytes_ = 0;
}

std::size_t device_bytes_current() { return mcc_device_bytes_current(); }
std::size_t device_bytes_peak() { return mcc_device_bytes_peak(); }
void device_bytes_reset_peak() { mcc_device_bytes_reset_peak(); }

Storage::Storage(Backend& backend, std::size_t bytes) : nbytes(bytes) {
    (void)backend;
    MCL_CHECK(bytes > 0, "cannot allocate zero-byte buffer");
    MCL_CHECK(mcc_device_alloc(&hip_ptr, bytes) == MCC_OK, std::string("device allocation failed: ") + mcc_last_error());
}

Storage::~Storage() {
    if (hip_ptr) mcc_device_free(hip_ptr);
}

void clear_memory_pool() { mcc_device_pool_clear(); }

}  // namespace motifcl
