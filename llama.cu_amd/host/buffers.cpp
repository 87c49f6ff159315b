// mapped_buffer, scoped_gpu, gpu_buffer_view, gpu_buffer: behaviour of llama_cu.cu:542-736.
#include <assert.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <unistd.h>

#include <utility>

#include "host_common.hpp"

namespace llama_cu {

mapped_buffer::mapped_buffer() {}

// existing file, read-only, private mapping (llama_cu.cu:550-578)
mapped_buffer::mapped_buffer(std::string const& path) {
  fd_ = open(path.c_str(), O_RDONLY);
  if (fd_ < 0) {
    return;
  }
  off_t end = lseek(fd_, 0, SEEK_END);
  if (end < 0) {
    return;
  }
  size_ = (size_t)end;
  void* p = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
  ptr_ = (p == MAP_FAILED) ? nullptr : p;
}

// new (or truncated) file of `size` bytes, shared read/write mapping (llama_cu.cu:579-611)
mapped_buffer::mapped_buffer(std::string const& path, size_t size) {
  fd_ = open(path.c_str(), O_RDWR | O_CREAT | O_TRUNC, 0644);
  if (fd_ < 0) {
    return;
  }
  size_ = size;
  if (ftruncate(fd_, (off_t)size_) < 0) {
    close(fd_);
    fd_ = -1;
    return;
  }
  void* p = mmap(nullptr, size_, PROT_READ | PROT_WRITE, MAP_SHARED, fd_, 0);
  ptr_ = (p == MAP_FAILED) ? nullptr : p;
}

// anonymous memory (llama_cu.cu:612-628)
mapped_buffer::mapped_buffer(size_t size) {
  size_ = size;
  void* p = mmap(nullptr, size_, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
  ptr_ = (p == MAP_FAILED) ? nullptr : p;
}

void mapped_buffer::release() {
  if (ptr_) {
    munmap(ptr_, size_);
  }
  if (fd_ >= 0) {
    close(fd_);
  }
  fd_ = -1;
  ptr_ = nullptr;
  size_ = 0;
}

mapped_buffer::~mapped_buffer() { release(); }

mapped_buffer::mapped_buffer(mapped_buffer&& other)
    : fd_(std::exchange(other.fd_, -1)), ptr_(std::exchange(other.ptr_, nullptr)), size_(std::exchange(other.size_, 0)) {}

mapped_buffer& mapped_buffer::operator=(mapped_buffer&& other) {
  if (this != &other) {
    release();
    fd_ = std::exchange(other.fd_, -1);
    ptr_ = std::exchange(other.ptr_, nullptr);
    size_ = std::exchange(other.size_, 0);
  }
  return *this;
}

scoped_gpu::scoped_gpu(int device) {
  LCU_CHECK(lcu_get_device(&prev_device_));
  LCU_CHECK(lcu_set_device(device));
}
scoped_gpu::~scoped_gpu() { LCU_CHECK(lcu_set_device(prev_device_)); }

void gpu_buffer_view::copy_from(mapped_buffer const& buffer) {
  assert(buffer.size() == size_);
  LCU_CHECK(lcu_h2d(dev_ptr_, buffer.data(), buffer.size(), nullptr));
}
void gpu_buffer_view::copy_from(void const* buffer, size_t size) {
  assert(size <= size_);
  LCU_CHECK(lcu_h2d(dev_ptr_, buffer, size, nullptr));
}
void gpu_buffer_view::copy_to(void* buffer, size_t size) {
  assert(size <= size_);
  LCU_CHECK(lcu_d2h(buffer, dev_ptr_, size, nullptr));
}

gpu_buffer::gpu_buffer(size_t size) {
  device_structure_lock lock(device_structure_mutex());
  LCU_CHECK(lcu_malloc(&dev_ptr_, size));
  size_ = size;
}
gpu_buffer::gpu_buffer(gpu_buffer&& other) : gpu_buffer_view(other.dev_ptr_, other.size_) {
  other.dev_ptr_ = nullptr;
  other.size_ = 0;
}
gpu_buffer& gpu_buffer::operator=(gpu_buffer&& other) {
  if (this != &other) {
    if (dev_ptr_) {
      device_structure_lock lock(device_structure_mutex());
      LCU_CHECK(lcu_free(dev_ptr_));
    }
    dev_ptr_ = std::exchange(other.dev_ptr_, nullptr);
    size_ = std::exchange(other.size_, 0);
  }
  return *this;
}
gpu_buffer::~gpu_buffer() {
  if (dev_ptr_) {
    device_structure_lock lock(device_structure_mutex());
    LCU_CHECK(lcu_free(dev_ptr_));
  }
}

}  // namespace llama_cu
