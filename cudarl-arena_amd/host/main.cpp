// Demo equal to the reference's src/main.cu:21-99 without the 500 ms sleeps:
// ten random steps of one Environment, then one CudaQLearning::update_batch.
#include <cstdlib>
#include <iostream>
#include <utility>
#include <vector>

#include "environment.h"
#include "q_learning.h"

int main() {
  std::cout << "=== CudaRL-Arena: MI355X-accelerated Reinforcement Learning ===" << std::endl;
  Environment env(0);
  CudaQLearning q_learning(env.getWidth(), env.getHeight(), 4, 0.1f, 0.99f);
  env.reset();

  std::vector<std::pair<int, int>> states, next_states;
  std::vector<int> actions;
  std::vector<float> rewards;
  std::vector<bool> dones;
  for (int step = 0; step < 10; step++) {
    const int x = env.getAgentX(), y = env.getAgentY();
    const int action = std::rand() % 4;
    std::cout << "Step " << step << ": Agent at (" << x << "," << y << "), action " << action << std::endl;
    states.push_back({x, y});
    actions.push_back(action);
    env.step(action);
    rewards.push_back(env.getReward());
    next_states.push_back({env.getAgentX(), env.getAgentY()});
    dones.push_back(env.isDone());
    std::cout << "  New position: (" << env.getAgentX() << "," << env.getAgentY() << "), Reward: "
              << env.getReward() << ", Done: " << (env.isDone() ? "true" : "false") << std::endl;
    if (env.isDone()) break;
  }
  q_learning.update_batch(states, actions, rewards, next_states, dones);
  std::cout << "\nSample Q-values after update:" << std::endl;
  for (int a = 0; a < 4; a++)
    std::cout << "  Q(0,0," << a << ") = " << q_learning.get_q_value(0, 0, a) << std::endl;
  return 0;
}
