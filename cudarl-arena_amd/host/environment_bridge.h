// EnvironmentBridge: the gym-shaped wrapper the reference exposes to Python
// (src/environment_bridge.h:10-80), same signatures.  addObstacle / setGoal /
// addTrap only print upstream (src/environment_bridge.cu:53-78); here they edit
// the map.
#pragma once
#include <memory>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "environment.h"

class EnvironmentBridge {
 public:
  EnvironmentBridge(int width = 10, int height = 10);

  std::vector<float> reset();
  std::tuple<std::vector<float>, float, bool, std::string> step(int action);
  std::vector<float> getObservation() const;
  int getWidth() const;
  int getHeight() const;
  std::pair<int, int> getAgentPosition() const;
  void addObstacle(int x, int y);
  void setGoal(int x, int y);
  void addTrap(int x, int y, float penalty = -1.0f);

 private:
  std::unique_ptr<Environment> env;
  int width;
  int height;
};
