// Minimal command-line flags with the gflags surface the reference's main uses
// (DEFINE_bool/int32/double/string, DECLARE_*, FLAGS_name, ParseCommandLineFlags; src/main.cu:32-109).
// gflags itself is an empty, un-vendored submodule of the reference, so the parser is written here.
// Accepted forms: --name=value, --name value, -name=value, -name value, --name / --noname for booleans.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>

namespace skyflags {

struct Flag {
  enum Kind { BOOL, INT32, DOUBLE, STRING } kind;
  void* ptr;
  const char* help;
};
inline std::map<std::string, Flag>& registry() {
  static std::map<std::string, Flag> r;
  return r;
}
struct Registrar {
  Registrar(const char* name, Flag::Kind k, void* p, const char* help) { registry()[name] = Flag{k, p, help}; }
};

inline bool parse_bool(const std::string& v, bool* out) {
  if (v == "1" || v == "true" || v == "t" || v == "yes" || v == "y") { *out = true; return true; }
  if (v == "0" || v == "false" || v == "f" || v == "no" || v == "n") { *out = false; return true; }
  return false;
}

inline bool set_flag(const std::string& name, const std::string& value) {
  auto it = registry().find(name);
  if (it == registry().end()) return false;
  Flag& f = it->second;
  char* end = nullptr;
  switch (f.kind) {
    case Flag::BOOL: return parse_bool(value, static_cast<bool*>(f.ptr));
    case Flag::INT32: {
      long v = strtol(value.c_str(), &end, 10);
      if (!end || *end) return false;
      *static_cast<int32_t*>(f.ptr) = (int32_t)v;
      return true;
    }
    case Flag::DOUBLE: {
      double v = strtod(value.c_str(), &end);
      if (!end || *end) return false;
      *static_cast<double*>(f.ptr) = v;
      return true;
    }
    case Flag::STRING: *static_cast<std::string*>(f.ptr) = value; return true;
  }
  return false;
}

// Returns 0 on success; prints the offending flag and returns 1 otherwise (gflags exits with 1).
inline int ParseCommandLineFlags(int* argc, char*** argv) {
  for (int i = 1; i < *argc; ++i) {
    std::string a = (*argv)[i];
    if (a.size() < 2 || a[0] != '-') {
      fprintf(stderr, "ERROR: unexpected argument '%s'\n", a.c_str());
      return 1;
    }
    a = a.substr(a[1] == '-' ? 2 : 1);
    std::string name = a, value;
    bool has_value = false;
    const size_t eq = a.find('=');
    if (eq != std::string::npos) {
      name = a.substr(0, eq);
      value = a.substr(eq + 1);
      has_value = true;
    }
    auto it = registry().find(name);
    if (it == registry().end() && !has_value && name.rfind("no", 0) == 0) {
      auto neg = registry().find(name.substr(2));
      if (neg != registry().end() && neg->second.kind == Flag::BOOL) {
        *static_cast<bool*>(neg->second.ptr) = false;
        continue;
      }
    }
    if (it == registry().end()) {
      fprintf(stderr, "ERROR: unknown command line flag '%s'\n", name.c_str());
      return 1;
    }
    if (!has_value) {
      if (it->second.kind == Flag::BOOL) {
        bool b;
        if (i + 1 < *argc && parse_bool((*argv)[i + 1], &b) && (*argv)[i + 1][0] != '-') {
          value = (*argv)[++i];
        } else {
          value = "true";
        }
      } else {
        if (i + 1 >= *argc) {
          fprintf(stderr, "ERROR: flag '%s' is missing its argument\n", name.c_str());
          return 1;
        }
        value = (*argv)[++i];
      }
    }
    if (!set_flag(name, value)) {
      fprintf(stderr, "ERROR: illegal value '%s' specified for flag '%s'\n", value.c_str(), name.c_str());
      return 1;
    }
  }
  return 0;
}

}  // namespace skyflags

#define DEFINE_bool(name, val, txt) \
  bool FLAGS_##name = val;          \
  static skyflags::Registrar reg_##name(#name, skyflags::Flag::BOOL, &FLAGS_##name, txt)
#define DEFINE_int32(name, val, txt) \
  int32_t FLAGS_##name = val;        \
  static skyflags::Registrar reg_##name(#name, skyflags::Flag::INT32, &FLAGS_##name, txt)
#define DEFINE_double(name, val, txt) \
  double FLAGS_##name = val;          \
  static skyflags::Registrar reg_##name(#name, skyflags::Flag::DOUBLE, &FLAGS_##name, txt)
#define DEFINE_string(name, val, txt) \
  std::string FLAGS_##name = val;     \
  static skyflags::Registrar reg_##name(#name, skyflags::Flag::STRING, &FLAGS_##name, txt)
#define DECLARE_bool(name) extern bool FLAGS_##name
#define DECLARE_int32(name) extern int32_t FLAGS_##name
#define DECLARE_double(name) extern double FLAGS_##name
#define DECLARE_string(name) extern std::string FLAGS_##name
