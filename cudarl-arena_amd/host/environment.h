// Environment: the reference's single-grid host class (src/environment.h:17-47)
// on top of the batched HIP engine's C ABI with n_envs = 1.  Public signatures
// are the reference's; everything else is private or additive.
#pragma once
#include <cstdint>
#include <vector>

struct crl_engine;

// Mirror of the reference's POD (src/environment.h:7-15).  `grid` points into
// host memory owned by the Environment; the device keeps 2-bit cell classes.
struct EnvironmentState {
  int width;
  int height;
  float* grid;
  int agent_x;
  int agent_y;
  float reward;
  bool done;
};

class Environment {
 public:
  Environment(int id = 0, int width = 10, int height = 10);
  ~Environment();
  // two device allocations behind one handle: moving is fine, copying is not
  // (the reference forgets to delete these and would double-free)
  Environment(const Environment&) = delete;
  Environment& operator=(const Environment&) = delete;
  Environment(Environment&& other) noexcept;
  Environment& operator=(Environment&& other) noexcept;

  void reset();
  void step(int action);

  int getWidth() const { return state.width; }
  int getHeight() const { return state.height; }
  int getAgentX() const { return state.agent_x; }
  int getAgentY() const { return state.agent_y; }
  float getReward() const { return state.reward; }
  bool isDone() const { return state.done; }

  float getCellValue(int x, int y) const;
  std::vector<float> getGrid() const;

  // Additive: write one cell of the float grid.  The value is classified with
  // the thresholds of src/kernels.cu:30-63 unless `trap` forces a TRAP cell
  // whose bump penalty is the value itself (so a penalty of exactly -1.0f works).
  void setCellValue(int x, int y, float value, bool trap = false);

 private:
  int env_id;
  EnvironmentState state;
  crl_engine* engine;
  std::vector<float> grid_store;

  void initializeGrid();
  void updateHostState();
  void release() noexcept;
};
