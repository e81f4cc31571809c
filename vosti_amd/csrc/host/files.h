// Reading small text files, for config.json, generation_config.json and the index of a sharded checkpoint.
#pragma once
#include <sys/stat.h>

#include <fstream>
#include <sstream>
#include <stdexcept>
#include <string>

namespace vosti {

struct FileError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline std::string read_text_file(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) throw FileError("cannot read " + path);
  std::ostringstream s;
  s << f.rdbuf();
  return s.str();
}

inline bool file_exists(const std::string& path) {
  struct stat st;
  return stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

}  // namespace vosti
