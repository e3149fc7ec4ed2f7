// Host memory providers of the ShmTensorLib surface: POSIX shared-memory
// segments, memory-mapped .npy files and the tensors that view them
// (include/shm_memory.h:6-57, include/utils.h:5-13, src/mmap_tensor.cc:10-57,
// src/cnpy.cc:9-87 in the ShmTensor tree). Host code only. With
// pin_memory=true the mapped range is registered in place for GPU access
// (shmt_host_register); failures raise RuntimeError instead of aborting.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <torch/extension.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>
#include <fstream>
#include <string>
#include <tuple>
#include <vector>

#include "shmt.h"

namespace py = pybind11;

namespace shim {
bool host_register_enabled();  // module.cc: the opt-in switch for registering existing memory in place
}

namespace {

// Registers a fresh mapping for GPU access, where that is switched on.
// Registering memory that already exists is refused by some drivers, and a
// refused call can leave its error for the next HIP call to report, so the
// runtime is only asked when in-place registration was requested
// (set_host_register(True) / SHMT_HOST_REGISTER=1, the switch pin_memory()
// honours too). Without the request, or when the driver refuses, the mapping is
// taken down again (and the segment this call created removed) before the
// error is raised, so a refused request leaves nothing behind.
void pin_range(void *ptr, int64_t size, int fd, const char *what, const char *unlink_name) {
  const bool asked = shim::host_register_enabled();
  if (asked && shmt_host_register(ptr, size) == SHMT_OK) return;
  const std::string why = asked ? std::string("the driver refused: ") + shmt_last_error()
                                : std::string("in-place registration is switched off; set_host_register(True) or "
                                              "SHMT_HOST_REGISTER=1 asks the driver for it");
  munmap(ptr, static_cast<size_t>(size));
  close(fd);
  if (unlink_name != nullptr) shm_unlink(unlink_name);
  TORCH_CHECK(false, what, "(pin_memory=True): the existing mapping was not registered for GPU access (",
              why, "). Open it with pin_memory=False and hand the GPU operators a staging copy in pinned "
              "memory instead: `staged = obj.pinned()` on a ShmTensor / DiskTensor (`obj.flush()` copies it "
              "back into the mapping), or `tensor.pin_memory()` on the plain tensor.");
}

void *map_fd(int fd, int64_t size, const std::string &name) {
  void *ptr = mmap(nullptr, static_cast<size_t>(size), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (ptr == MAP_FAILED) {
    const int err = errno;
    close(fd);
    TORCH_CHECK(false, "failed to map ", name, ": ", strerror(err));
  }
  return ptr;
}

// include/shm_memory.h:6-23
std::tuple<int64_t, int64_t> create_shared_mem(const std::string &name, int64_t size,
                                               bool pin_memory) {
  TORCH_CHECK(size > 0, "create_shared_mem: size must be positive");
  const int fd = shm_open(name.c_str(), O_RDWR | O_CREAT, S_IRUSR | S_IWUSR);
  TORCH_CHECK(fd != -1, "fail to open ", name, ": ", strerror(errno));
  if (ftruncate(fd, static_cast<off_t>(size)) == -1) {
    const int err = errno;
    close(fd);
    shm_unlink(name.c_str());
    TORCH_CHECK(false, "Failed to truncate the file. ", strerror(err));
  }
  void *ptr = map_fd(fd, size, name);
  if (pin_memory) pin_range(ptr, size, fd, "create_shared_mem", name.c_str());
  return std::make_tuple(reinterpret_cast<int64_t>(ptr), static_cast<int64_t>(fd));
}

// include/shm_memory.h:25-39
std::tuple<int64_t, int64_t> open_shared_mem(const std::string &name, int64_t size,
                                             bool pin_memory) {
  TORCH_CHECK(size > 0, "open_shared_mem: size must be positive");
  const int fd = shm_open(name.c_str(), O_RDWR, S_IRUSR | S_IWUSR);
  TORCH_CHECK(fd != -1, "fail to open ", name, ": ", strerror(errno));
  void *ptr = map_fd(fd, size, name);
  if (pin_memory) pin_range(ptr, size, fd, "open_shared_mem", nullptr);
  return std::make_tuple(reinterpret_cast<int64_t>(ptr), static_cast<int64_t>(fd));
}

// include/shm_memory.h:41-49
void release_shared_mem(const std::string &name, int64_t size, int64_t ptr, int64_t fd,
                        bool pin_memory) {
  void *p = reinterpret_cast<void *>(ptr);
  if (pin_memory) TORCH_CHECK(shmt_host_unregister(p) == SHMT_OK, shmt_last_error());
  TORCH_CHECK(munmap(p, static_cast<size_t>(size)) != -1, strerror(errno));
  close(static_cast<int>(fd));
  shm_unlink(name.c_str());
}

// include/shm_memory.h:51-56
torch::Tensor open_shared_tensor(int64_t ptr, py::object dtype, std::vector<int64_t> shape) {
  const torch::ScalarType type = torch::python::detail::py_object_to_dtype(dtype);
  return torch::from_blob(reinterpret_cast<void *>(ptr), shape, torch::TensorOptions().dtype(type));
}

// include/utils.h:5-13: does a shared-memory segment of that name exist?
bool file_exist(const std::string &filename) {
  const int fd = shm_open(filename.c_str(), O_RDONLY, S_IRUSR | S_IWUSR);
  if (fd < 0) return false;
  close(fd);
  return true;
}

struct NpyHeader {
  torch::ScalarType dtype;
  std::vector<int64_t> shape;
  int64_t offset;
  bool fortran_order;
};

// .npy header: magic "\x93NUMPY", version (major, minor), little-endian
// header length (2 bytes for version 1, 4 bytes for 2 and 3), then a Python
// dict literal with 'descr', 'fortran_order' and 'shape'. The dtype table is
// the reference's (src/cnpy.cc:9-14).
NpyHeader parse_npy_header(const std::string &fname) {
  std::ifstream in(fname, std::ios::binary);
  TORCH_CHECK(in.good(), "npy_load: Unable to open file ", fname);
  unsigned char pre[12] = {0};
  in.read(reinterpret_cast<char *>(pre), 10);
  TORCH_CHECK(in.gcount() == 10 && pre[0] == 0x93 && std::memcmp(pre + 1, "NUMPY", 5) == 0,
              "parse_npy_header: ", fname, " is not a .npy file");
  const int major = pre[6];
  size_t header_len = 0, header_start = 0;
  if (major == 1) {
    header_len = pre[8] | (static_cast<size_t>(pre[9]) << 8);
    header_start = 10;
  } else {
    in.read(reinterpret_cast<char *>(pre + 10), 2);
    TORCH_CHECK(in.gcount() == 2, "parse_npy_header: truncated header");
    header_len = pre[8] | (static_cast<size_t>(pre[9]) << 8) | (static_cast<size_t>(pre[10]) << 16) |
                 (static_cast<size_t>(pre[11]) << 24);
    header_start = 12;
  }
  std::string header(header_len, '\0');
  in.read(&header[0], static_cast<std::streamsize>(header_len));
  TORCH_CHECK(static_cast<size_t>(in.gcount()) == header_len, "parse_npy_header: truncated header");

  NpyHeader h;
  h.offset = static_cast<int64_t>(header_start + header_len);

  size_t loc = header.find("fortran_order");
  TORCH_CHECK(loc != std::string::npos, "parse_npy_header: failed to find header keyword: 'fortran_order'");
  loc = header.find(':', loc);
  TORCH_CHECK(loc != std::string::npos, "parse_npy_header: malformed 'fortran_order'");
  h.fortran_order = header.find("True", loc) != std::string::npos &&
                    header.find("True", loc) < header.find_first_of(",}", loc);

  loc = header.find("shape");
  TORCH_CHECK(loc != std::string::npos, "parse_npy_header: failed to find header keyword: 'shape'");
  const size_t open = header.find('(', loc), close = header.find(')', loc);
  TORCH_CHECK(open != std::string::npos && close != std::string::npos && open < close,
              "parse_npy_header: failed to find header keyword: '(' or ')'");
  int64_t cur = -1;
  for (size_t i = open + 1; i < close; ++i) {
    const char c = header[i];
    if (c >= '0' && c <= '9') {
      cur = (cur < 0 ? 0 : cur) * 10 + (c - '0');
    } else if (cur >= 0) {
      h.shape.push_back(cur);
      cur = -1;
    }
  }
  if (cur >= 0) h.shape.push_back(cur);

  loc = header.find("descr");
  TORCH_CHECK(loc != std::string::npos, "parse_npy_header: failed to find header keyword: 'descr'");
  loc = header.find(':', loc);
  const size_t q0 = header.find('\'', loc);
  const size_t q1 = q0 == std::string::npos ? q0 : header.find('\'', q0 + 1);
  TORCH_CHECK(q0 != std::string::npos && q1 != std::string::npos, "parse_npy_header: malformed 'descr'");
  const std::string descr = header.substr(q0 + 1, q1 - q0 - 1);
  static const std::pair<const char *, torch::ScalarType> kTypes[] = {
      {"<f2", torch::kFloat16}, {"<f4", torch::kFloat32}, {"<f8", torch::kFloat64},
      {"|u1", torch::kUInt8},   {"|i1", torch::kInt8},    {"<i2", torch::kInt16},
      {"<i4", torch::kInt32},   {"<i8", torch::kInt64},
  };
  bool found = false;
  for (const auto &t : kTypes) {
    if (descr == t.first) {
      h.dtype = t.second;
      found = true;
    }
  }
  TORCH_CHECK(found, "parse_npy_header: failed to find dtype ", descr);
  return h;
}

// src/mmap_tensor.cc:10-47: returns (tensor, mapped size, mapping address, fd).
std::tuple<torch::Tensor, int64_t, int64_t, int64_t> open_mmap_tensor(const std::string &fname,
                                                                      bool pin_memory) {
  const NpyHeader h = parse_npy_header(fname);
  TORCH_CHECK(!h.fortran_order, "fortran order is not supported");
  const int fd = open(fname.c_str(), O_RDWR, S_IRUSR | S_IWUSR);
  TORCH_CHECK(fd != -1, "open file failed: ", fname);
  const int64_t file_size = static_cast<int64_t>(lseek(fd, 0, SEEK_END));
  int64_t need = static_cast<int64_t>(c10::elementSize(h.dtype));
  for (int64_t d : h.shape) need *= d;
  if (file_size < h.offset + need) {
    close(fd);
    TORCH_CHECK(false, fname, ": file is shorter than its header says");
  }
  void *ptr = map_fd(fd, file_size, fname);
  // the whole file is registered, the tensor starts at ptr + offset (src/mmap_tensor.cc:39-45)
  if (pin_memory) pin_range(ptr, file_size, fd, "open_mmap_tensor", nullptr);
  torch::Tensor tensor = torch::from_blob(static_cast<char *>(ptr) + h.offset, h.shape,
                                          torch::TensorOptions().dtype(h.dtype));
  return std::make_tuple(tensor, file_size, reinterpret_cast<int64_t>(ptr), static_cast<int64_t>(fd));
}

// src/mmap_tensor.cc:49-55
void close_mmap_tensor(int64_t size, int64_t ptr, int64_t fd, bool pin_memory) {
  void *p = reinterpret_cast<void *>(ptr);
  if (pin_memory) TORCH_CHECK(shmt_host_unregister(p) == SHMT_OK, shmt_last_error());
  TORCH_CHECK(munmap(p, static_cast<size_t>(size)) != -1, strerror(errno));
  close(static_cast<int>(fd));
}

}  // namespace

// Names, keyword names and defaults of src/pybind.cc:17-30.
void register_host_tensors(py::module &m) {
  m.def("create_shared_mem", &create_shared_mem, py::arg("name"), py::arg("size"),
        py::arg("pin_memory") = false)
      .def("open_shared_mem", &open_shared_mem, py::arg("name"), py::arg("size"),
           py::arg("pin_memory") = false)
      .def("release_shared_mem", &release_shared_mem, py::arg("name"), py::arg("size"),
           py::arg("ptr"), py::arg("fd"), py::arg("pin_memory") = false)
      .def("open_shared_tensor", &open_shared_tensor, py::arg("ptr"), py::arg("dtype"),
           py::arg("shape"))
      .def("file_exist", &file_exist, py::arg("filename"))
      .def("open_mmap_tensor", &open_mmap_tensor, py::arg("filename"), py::arg("pin_memory"))
      .def("close_mmap_tensor", &close_mmap_tensor, py::arg("size"), py::arg("ptr"), py::arg("fd"),
           py::arg("pin_memory"));
}
