// Minimal .npy (format 1.0) reader / writer for Q-tables, and the conversion
// between the engine's fp32 layout Q[(y*W + x)*A + a] (src/q_learning.cu:196)
// and the reference agent's float64 array of shape (W, H, A) indexed [x, y, a]
// that QTableAgent.save / load exchange with np.save / np.load
// (src/train.py:63,150-168; read back by src/visualize.py:299-302).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace crl_npy {

struct Array {
  std::vector<int64_t> shape;
  bool is_double = false;        // '<f8' (else '<f4')
  std::vector<double> f64;       // filled when is_double
  std::vector<float> f32;        // filled otherwise
};

// throws std::runtime_error on I/O errors or unsupported files (only C-order
// little-endian float32 / float64 arrays are understood)
Array load(const std::string& path);
void save_f32(const std::string& path, const std::vector<int64_t>& shape, const float* data);
void save_f64(const std::string& path, const std::vector<int64_t>& shape, const double* data);

// engine layout (S*A floats) -> reference layout: float64 (W, H, A), [x, y, a]
std::vector<double> to_reference_layout(const std::vector<float>& q, int width, int height, int actions);
// and back; accepts a float64 or float32 array of shape (W, H, A)
std::vector<float> from_reference_layout(const Array& a, int width, int height, int actions);

// QTableAgent.save / load (src/train.py:150-168)
void save_agent(const std::string& path, const std::vector<float>& q, int width, int height, int actions);
std::vector<float> load_agent(const std::string& path, int width, int height, int actions);

}  // namespace crl_npy
