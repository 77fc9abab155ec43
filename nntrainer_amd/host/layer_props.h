// SPDX-License-Identifier: Apache-2.0
/**
 * @file   layer_props.h
 * @brief  "key=value" property parsing for the HIP layers.
 *
 * The framework's layers parse properties with loadProperties() into typed
 * tuples and hand what is left to LayerImpl::setProperty, which rejects unknown
 * keys (nntrainer/layers/layer_impl.cpp). These layers derive from Layer
 * directly, so the same contract is kept here in a few lines: keys are case
 * insensitive, a value is everything after the first '=', an unknown key is a
 * std::invalid_argument.
 */
#ifndef HIPQ_LAYER_PROPS_H
#define HIPQ_LAYER_PROPS_H

#include <algorithm>
#include <cctype>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace hipq_host {

inline std::string lower(std::string s) {
  std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::tolower(c); });
  return s;
}

inline std::string trim(const std::string &s) {
  size_t b = 0, e = s.size();
  while (b < e && std::isspace((unsigned char)s[b]))
    ++b;
  while (e > b && std::isspace((unsigned char)s[e - 1]))
    --e;
  return s.substr(b, e - b);
}

/** splits "key = value" entries; throws on an entry without '=' or an empty side */
inline std::vector<std::pair<std::string, std::string>>
split_properties(const std::vector<std::string> &values) {
  std::vector<std::pair<std::string, std::string>> out;
  for (const auto &v : values) {
    const size_t eq = v.find('=');
    if (eq == std::string::npos)
      throw std::invalid_argument("property is not of the form key=value: " + v);
    std::string key = lower(trim(v.substr(0, eq))), val = trim(v.substr(eq + 1));
    if (key.empty() || val.empty())
      throw std::invalid_argument("property has an empty key or value: " + v);
    out.emplace_back(key, val);
  }
  return out;
}

inline bool parse_bool(const std::string &key, const std::string &v) {
  const std::string s = lower(v);
  if (s == "true" || s == "1")
    return true;
  if (s == "false" || s == "0")
    return false;
  throw std::invalid_argument("property " + key + " is not a boolean: " + v);
}

inline unsigned int parse_positive(const std::string &key, const std::string &v) {
  size_t pos = 0;
  long n = 0;
  try {
    n = std::stol(v, &pos);
  } catch (const std::exception &) {
    pos = 0;
  }
  if (pos != v.size() || n <= 0)
    throw std::invalid_argument("property " + key + " must be a positive integer: " + v);
  return (unsigned int)n;
}

} // namespace hipq_host

#endif /* HIPQ_LAYER_PROPS_H */
