// Host-side helpers of the engine that need no device: configuration checks,
// epsilon tables, 2-bit map packing.
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/crl.h"

namespace crl {

// The calling thread's last failure text, behind crl_last_error().
std::string& last_error();
// Notes `why` as the thread's last failure and returns `code`.
int fail_with(int code, const char* why);

// CRL_OK, or a negative status with the reason in `why`
int validate_config(const crl_config* cfg, std::string& why);

// Epsilon per global step (STEP_MULT) or per episode (EPISODE_*): the values a
// Python float would take under `eps *= decay` (src/train.py:140-141), i.e.
// doubles, rounded to fp32 once.
std::vector<float> build_eps_table(const crl_config& cfg);

// 16 cells per word, cell c in bits [2*(c%16), 2*(c%16)+1] of word c/16
void pack_classes(const uint8_t* cls, size_t n_cells, uint32_t* words);

}  // namespace crl
