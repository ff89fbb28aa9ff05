// Result of KNOperator::profile (reference include/mirage/profile_result.h:22-28).
#pragma once

namespace mirage {

struct ProfileResult {
  static int const NUM_WARPUP_ITERATIONS = 1024;
  static int const NUM_ITERATIONS = 1024;
  float run_time;  // mean milliseconds per launch

  static ProfileResult infinity();
};

}  // namespace mirage
