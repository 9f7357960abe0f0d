// Minimal JSON document reader for oneDNN-Graph partition strings.
// Objects keep their key order; integers that fit int64 are kept exact (the
// schema marks an unranked tensor with shape [INT64_MIN]).
#pragma once
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace gcapi {

struct JValue {
  enum Type { Null, Bool, Num, Str, Arr, Obj } type = Null;
  bool b = false;
  double num = 0;
  int64_t inum = 0;
  bool is_int = false;
  std::string str;
  std::vector<JValue> arr;
  std::vector<std::pair<std::string, JValue>> obj;
  const JValue *find(const std::string &k) const {
    for (auto &kv : obj)
      if (kv.first == k)
        return &kv.second;
    return nullptr;
  }
};

// throws std::invalid_argument on malformed input
JValue parse_json(const std::string &text);

} // namespace gcapi
