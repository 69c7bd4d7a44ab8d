#include "npy.h"

#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <stdexcept>

namespace crl_npy {
namespace {

const char kMagic[] = "\x93NUMPY";

std::string header_text(const char* descr, const std::vector<int64_t>& shape) {
  std::ostringstream h;
  h << "{'descr': '" << descr << "', 'fortran_order': False, 'shape': (";
  for (size_t i = 0; i < shape.size(); ++i) h << shape[i] << (shape.size() == 1 || i + 1 < shape.size() ? ", " : "");
  h << "), }";
  std::string s = h.str();
  // magic(6) + version(2) + length(2) + header, padded with spaces to a multiple of 64, ending in '\n'
  const size_t unpadded = 10 + s.size() + 1;
  s.append((64 - unpadded % 64) % 64, ' ');
  s.push_back('\n');
  return s;
}

void write_file(const std::string& path, const char* descr, const std::vector<int64_t>& shape,
                const void* data, size_t bytes) {
  const std::string h = header_text(descr, shape);
  std::ofstream f(path, std::ios::binary);
  if (!f) throw std::runtime_error("cannot open " + path + " for writing");
  f.write(kMagic, 6);
  const unsigned char ver[2] = {1, 0};
  f.write(reinterpret_cast<const char*>(ver), 2);
  const unsigned char len[2] = {(unsigned char)(h.size() & 0xff), (unsigned char)(h.size() >> 8)};
  f.write(reinterpret_cast<const char*>(len), 2);
  f.write(h.data(), (std::streamsize)h.size());
  f.write(static_cast<const char*>(data), (std::streamsize)bytes);
  if (!f) throw std::runtime_error("write to " + path + " failed");
}

size_t count(const std::vector<int64_t>& shape) {
  size_t n = 1;
  for (int64_t d : shape) n *= (size_t)d;
  return n;
}

}  // namespace

void save_f32(const std::string& path, const std::vector<int64_t>& shape, const float* data) {
  write_file(path, "<f4", shape, data, count(shape) * sizeof(float));
}

void save_f64(const std::string& path, const std::vector<int64_t>& shape, const double* data) {
  write_file(path, "<f8", shape, data, count(shape) * sizeof(double));
}

Array load(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) throw std::runtime_error("cannot open " + path);
  char magic[6];
  unsigned char ver[2];
  f.read(magic, 6);
  f.read(reinterpret_cast<char*>(ver), 2);
  if (!f || std::memcmp(magic, kMagic, 6) != 0) throw std::runtime_error(path + " is not a .npy file");
  size_t hlen = 0;
  if (ver[0] == 1) {
    unsigned char l[2];
    f.read(reinterpret_cast<char*>(l), 2);
    hlen = (size_t)l[0] | ((size_t)l[1] << 8);
  } else if (ver[0] == 2 || ver[0] == 3) {
    unsigned char l[4];
    f.read(reinterpret_cast<char*>(l), 4);
    hlen = (size_t)l[0] | ((size_t)l[1] << 8) | ((size_t)l[2] << 16) | ((size_t)l[3] << 24);
  } else {
    throw std::runtime_error(path + ": unsupported .npy version");
  }
  // the header's length is checked against the file before it is allocated
  const std::streamoff h_at = f.tellg();
  f.seekg(0, std::ios::end);
  const std::streamoff h_left = f.tellg() - h_at;
  f.seekg(h_at);
  if (!f || h_left < 0 || hlen > (size_t)h_left) throw std::runtime_error(path + ": truncated header");
  std::string h(hlen, '\0');
  f.read(&h[0], (std::streamsize)hlen);
  if (!f) throw std::runtime_error(path + ": truncated header");
  Array a;
  if (h.find("'<f8'") != std::string::npos || h.find("'=f8'") != std::string::npos)
    a.is_double = true;
  else if (h.find("'<f4'") == std::string::npos && h.find("'=f4'") == std::string::npos)
    throw std::runtime_error(path + ": only little-endian float32 / float64 arrays are supported");
  if (h.find("'fortran_order': False") == std::string::npos)
    throw std::runtime_error(path + ": Fortran-ordered arrays are not supported");
  const size_t sp = h.find("'shape':");
  const size_t lp = h.find('(', sp), rp = h.find(')', lp);
  if (sp == std::string::npos || lp == std::string::npos || rp == std::string::npos)
    throw std::runtime_error(path + ": no shape in header");
  std::string dims = h.substr(lp + 1, rp - lp - 1);
  for (char& c : dims)
    if (c == ',') c = ' ';
  std::istringstream ds(dims);
  int64_t d;
  while (ds >> d) {
    if (d < 0) throw std::runtime_error(path + ": negative dimension in header");
    a.shape.push_back(d);
  }
  // the header's word is checked against the file before anything is allocated
  const std::streamoff at = f.tellg();
  f.seekg(0, std::ios::end);
  const std::streamoff left = f.tellg() - at;
  f.seekg(at);
  const size_t elem = a.is_double ? sizeof(double) : sizeof(float);
  const size_t max_elems = left > 0 ? (size_t)left / elem : 0;
  size_t n = 1;
  for (int64_t dim : a.shape)
    if (dim == 0) n = 0;  // an empty array, whatever the other dimensions say
  for (int64_t dim : a.shape) {
    if (n == 0) break;
    if (n > max_elems / (size_t)dim) throw std::runtime_error(path + ": truncated data");
    n *= (size_t)dim;
  }
  if (a.is_double) {
    a.f64.resize(n);
    f.read(reinterpret_cast<char*>(a.f64.data()), (std::streamsize)(n * sizeof(double)));
  } else {
    a.f32.resize(n);
    f.read(reinterpret_cast<char*>(a.f32.data()), (std::streamsize)(n * sizeof(float)));
  }
  if (!f) throw std::runtime_error(path + ": truncated data");
  return a;
}

std::vector<double> to_reference_layout(const std::vector<float>& q, int W, int H, int A) {
  if (q.size() != (size_t)W * H * A) throw std::runtime_error("Invalid Q-table size");
  std::vector<double> out(q.size());
  for (int x = 0; x < W; ++x)
    for (int y = 0; y < H; ++y)
      for (int a = 0; a < A; ++a)
        out[((size_t)x * H + y) * A + a] = (double)q[((size_t)y * W + x) * A + a];
  return out;
}

std::vector<float> from_reference_layout(const Array& arr, int W, int H, int A) {
  if (arr.shape.size() != 3 || arr.shape[0] != W || arr.shape[1] != H || arr.shape[2] != A)
    throw std::runtime_error("Invalid Q-table size");
  std::vector<float> q((size_t)W * H * A);
  for (int x = 0; x < W; ++x)
    for (int y = 0; y < H; ++y)
      for (int a = 0; a < A; ++a) {
        const size_t src = ((size_t)x * H + y) * A + a;
        q[((size_t)y * W + x) * A + a] = arr.is_double ? (float)arr.f64[src] : arr.f32[src];
      }
  return q;
}

void save_agent(const std::string& path, const std::vector<float>& q, int W, int H, int A) {
  const std::vector<double> ref = to_reference_layout(q, W, H, A);
  save_f64(path, {W, H, A}, ref.data());
}

std::vector<float> load_agent(const std::string& path, int W, int H, int A) {
  return from_reference_layout(load(path), W, H, A);
}

}  // namespace crl_npy
