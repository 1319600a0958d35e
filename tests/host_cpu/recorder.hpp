// What the recording launchers (stub_launch.cpp) leave for the test driver.
#pragma once

#include <string>
#include <vector>

namespace rec {
extern std::vector<std::string> log;             // one JSON object per launch, in issue order
extern std::string (*name_of)(const void *ptr);  // the driver's name for a device allocation
} // namespace rec
