// Driver for the CPU sanitizer leg (tests/test_sanitizers.py builds it with
// -fsanitize=address,undefined together with csrc/crl_host.cpp and host/npy.cpp and
// runs it): the host-only entry points of the C ABI - threaded map generators,
// epsilon tables, the float-grid classifier, Philox - and the .npy reader / writer,
// including files whose headers lie about their length or their shape.  Checks
// little itself: the point is that the sanitizers see every path run.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../include/crl.h"
#include "../cudarl-arena_amd/csrc/crl_host.h"
#include "../cudarl-arena_amd/host/npy.h"

#define REQUIRE(x)                                                         \
  do {                                                                     \
    if (!(x)) {                                                            \
      std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #x);  \
      std::exit(1);                                                        \
    }                                                                      \
  } while (0)

static void write_file(const std::string& path, const std::string& bytes) {
  std::ofstream f(path, std::ios::binary);
  f.write(bytes.data(), (std::streamsize)bytes.size());
}

static std::string npy_v1(const std::string& header_dict, size_t payload_bytes, int claim_len = -1) {
  std::string h = header_dict;
  while ((10 + h.size() + 1) % 64 != 0) h += ' ';
  h += '\n';
  const size_t len = claim_len >= 0 ? (size_t)claim_len : h.size();
  std::string out("\x93NUMPY\x01\x00", 8);
  out += (char)(len & 0xFF);
  out += (char)((len >> 8) & 0xFF);
  out += h;
  out += std::string(payload_bytes, '\x11');
  return out;
}

template <class F>
static bool throws(F&& f) {
  try {
    f();
  } catch (const std::runtime_error&) {
    return true;
  }
  return false;
}

int main(int argc, char** argv) {
  const std::string dir = argc > 1 ? argv[1] : "/tmp";

  // ---- map generators (they spread the maps over host threads) ----------------------
  {
    const int n = 301, W = 13, H = 7;  // sizes off every word and thread boundary
    std::vector<uint8_t> cls((size_t)n * W * H);
    std::vector<int32_t> start(n);
    REQUIRE(crl_gen_maps_bernoulli(7, n, n, W, H, 0.2f, 0.05f, cls.data(), start.data()) == CRL_OK);
    for (int i = 0; i < n; ++i) REQUIRE(start[i] >= 0 && start[i] < W * H && cls[(size_t)i * W * H + start[i]] == CRL_CELL_FREE);
    std::vector<uint8_t> one((size_t)W * H);
    std::vector<int32_t> starts(1000);
    REQUIRE(crl_gen_maps_bernoulli(8, 1, 1000, W, H, 0.15f, 0.0f, one.data(), starts.data()) == CRL_OK);
    REQUIRE(crl_gen_maps_bernoulli(8, 0, 10, W, H, 0.15f, 0.0f, one.data(), starts.data()) != CRL_OK);
    REQUIRE(!crl::last_error().empty());  // (crl_last_error() itself lives with the engine)
    // nearly everything a wall: the start / goal draws have few cells to choose from
    REQUIRE(crl_gen_maps_bernoulli(9, 5, 5, 4, 4, 0.8f, 0.1f, cls.data(), start.data()) == CRL_OK);

    const int m = 9, NW = 37, NH = 21;
    std::vector<uint8_t> ncls((size_t)m * NW * NH);
    std::vector<int32_t> nstart(m);
    std::vector<float> cr((size_t)m * NW * NH);
    REQUIRE(crl_gen_maps_noise(3, m, NW, NH, 8, 0.25f, 0.05f, 10.0f, ncls.data(), nstart.data(), cr.data()) == CRL_OK);
    REQUIRE(crl_gen_maps_noise(3, m, NW, NH, 0, 0.25f, 0.05f, 10.0f, ncls.data(), nstart.data(), cr.data()) != CRL_OK);
    size_t walls = 0;
    for (size_t i = 0; i < (size_t)NW * NH; ++i) walls += ncls[i] == CRL_CELL_WALL;
    REQUIRE(walls == (size_t)(0.25f * NW * NH));
  }

  // ---- epsilon tables, classifier, Philox ---------------------------------------------
  {
    crl_config c;
    std::memset(&c, 0, sizeof c);
    c.struct_size = sizeof c;
    c.n_envs = 4;
    c.width = 5;
    c.height = 5;
    c.n_actions = 4;
    c.auto_reset = 1;
    c.lr = 0.1f;
    c.gamma = 0.9f;
    c.eps0 = 1.0f;
    c.eps_decay = 0.995f;
    c.eps_end = 0.05f;
    c.eps_span = 100;
    for (int mode = 0; mode <= 3; ++mode) {
      c.eps_mode = mode;
      int32_t len = 0;
      REQUIRE(crl_eps_table(&c, nullptr, 0, &len) == CRL_OK && len >= 1);
      std::vector<float> tab((size_t)len);
      REQUIRE(crl_eps_table(&c, tab.data(), len, &len) == CRL_OK);
      std::vector<float> few(3, -1.0f);
      REQUIRE(crl_eps_table(&c, few.data(), 3, &len) == CRL_OK);  // a cap below the length copies the cap
      for (float e : tab) REQUIRE(e >= 0.0f && e <= 1.0f);
    }
    c.n_actions = 5;
    int32_t len = 0;
    REQUIRE(crl_eps_table(&c, nullptr, 0, &len) != CRL_OK);

    const float grid[] = {0.0f, 0.5f, 0.99f, 1.0f, -0.5f, -1.0f, -2.0f, -0.0f, NAN};
    uint8_t cls[9];
    float cr[9];
    REQUIRE(crl_classify_grid(grid, 9, -0.01f, cls, cr) == CRL_OK);
    REQUIRE(cls[0] == CRL_CELL_FREE && cls[2] == CRL_CELL_GOAL && cls[4] == CRL_CELL_TRAP && cls[5] == CRL_CELL_WALL);
    REQUIRE(crl_classify_grid(grid, 9, -0.01f, cls, nullptr) == CRL_OK);

    const uint32_t ctr[4] = {0, 0, 0, 0}, key[2] = {0, 0};
    uint32_t out[4];
    crl_philox4x32_10(ctr, key, out);
    REQUIRE(out[0] == 0x6627e8d5u && out[3] == 0x9b00dbd8u);
    float u;
    int32_t a;
    for (uint64_t t = 0; t < 64; ++t) {
      crl_explore_draw(~0ull, 0xFFFFFFFFu, ~0ull - t, 8, &u, &a);
      REQUIRE(u >= 0.0f && u < 1.0f && a >= 0 && a < 8);
    }
  }

  // ---- .npy reader / writer ---------------------------------------------------------------
  {
    const int W = 5, H = 3, A = 4;
    std::vector<float> q((size_t)W * H * A);
    for (size_t i = 0; i < q.size(); ++i) q[i] = (float)i * 0.25f - 3.0f;
    const std::string path = dir + "/sanitize_agent.npy";
    crl_npy::save_agent(path, q, W, H, A);
    REQUIRE(crl_npy::load_agent(path, W, H, A) == q);
    REQUIRE(throws([&] { crl_npy::load_agent(path, W + 1, H, A); }));
    crl_npy::save_f32(path, {H * W, A}, q.data());
    const crl_npy::Array arr = crl_npy::load(path);
    REQUIRE(!arr.is_double && arr.shape.size() == 2 && arr.f32 == q);
    crl_npy::save_f32(path, {}, q.data());  // a scalar
    REQUIRE(crl_npy::load(path).f32.size() == 1);

    const std::string dict = "{'descr': '<f4', 'fortran_order': False, 'shape': (5, 3, 4), }";
    write_file(path, npy_v1(dict, 240));
    REQUIRE(crl_npy::load(path).f32.size() == 60);
    write_file(path, npy_v1(dict, 239));                       // one byte short
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1(dict, 240, 60000));                // header longer than the file
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1(dict, 0, 3));                      // header cut inside the dictionary
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, std::string("\x93NUMPY\x02\x00\xff\xff\xff\xff", 12) + dict);  // version 2, 4 GB of header claimed
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, std::string("\x93NUMPY\x01", 7));         // cut inside the preamble
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1("{'descr': '<f4', 'fortran_order': False, 'shape': (4611686018427387904, 4611686018427387904, 16), }", 64));
    REQUIRE(throws([&] { crl_npy::load(path); }));             // the element count wraps around 2^64
    write_file(path, npy_v1("{'descr': '<f4', 'fortran_order': False, 'shape': (5, -3, 4), }", 240));
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1("{'descr': '<f4', 'fortran_order': False, 'shape': (5, 0, 4), }", 0));
    REQUIRE(crl_npy::load(path).f32.empty());
    write_file(path, npy_v1("{'descr': '<f4', 'fortran_order': False, 'shape': 5, 3", 240));  // no parentheses
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1("{'descr': '<i8', 'fortran_order': False, 'shape': (5,), }", 40));
    REQUIRE(throws([&] { crl_npy::load(path); }));
    write_file(path, npy_v1("{'descr': '<f8', 'fortran_order': True, 'shape': (5,), }", 40));
    REQUIRE(throws([&] { crl_npy::load(path); }));
    REQUIRE(throws([&] { crl_npy::load(dir + "/no_such_file.npy"); }));
    std::remove(path.c_str());
  }
  std::puts("sanitize_host ok");
  return 0;
}
