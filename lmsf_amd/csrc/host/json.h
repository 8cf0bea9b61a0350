// A small JSON reader for config.json: objects, arrays, strings, numbers, booleans and null into a tree.
// It keeps a number's text beside its value, so that a caller can tell 2 from 2.5 and report a value as written.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace lmsf {

struct Json {
  enum Kind { kNull, kBool, kNumber, kString, kArray, kObject };
  Kind kind = kNull;
  bool boolean = false;
  double number = 0.0;
  std::string text;                                   // a string's contents, or a number as it was written
  std::vector<Json> items;                            // array
  std::vector<std::pair<std::string, Json>> members;  // object, in the order written

  const Json* find(const std::string& key) const;     // member of an object, or null
  std::string repr() const;                            // the value as JSON text (strings in single quotes)
};

// Parses ``text``; throws lmsf::Error (kValueError) with the position of the first fault.
Json parse_json(const std::string& text);

}  // namespace lmsf
