// src/utils/params.h:4-5 restated: string-keyed scalar parameters handed to launchSampling.
#pragma once
#include <string>
#include <unordered_map>

using IntDict = std::unordered_map<std::string, int>;
using floatDict = std::unordered_map<std::string, float>;
