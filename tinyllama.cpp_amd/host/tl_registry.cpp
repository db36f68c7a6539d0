// tl_registry.cpp — see tl_registry.hpp.
#include "tl_registry.hpp"

#include <sys/stat.h>

#include <fstream>
#include <sstream>
#include <stdexcept>

#include "tl_gguf.hpp"
#include "tl_json.hpp"

namespace tlhost {

const std::vector<ModelFamily>& model_families() {
  static const std::vector<ModelFamily> table = {
      {"llama", "gguf", load_llama_gguf},
      {"Ralasun", "folder", load_stack_folder},
      {"Madalorn", "folder", load_stack_folder},
      {"Sogalix", "folder", load_stack_folder},
      {"Potipel", "folder", load_stack_folder},
  };
  return table;
}

const ModelFamily* find_model_family(const std::string& architecture, const std::string& container) {
  for (const ModelFamily& f : model_families())
    if (container == f.container && architecture == f.name) return &f;
  if (container == "gguf") return &model_families()[0];
  return nullptr;
}

std::string detect_architecture(const std::string& path, std::string* container, std::string* resolved) {
  struct stat st;
  if (stat(path.c_str(), &st) != 0) throw std::runtime_error("cannot open " + path);
  std::string cfg_path;
  if (S_ISDIR(st.st_mode)) {
    *resolved = path;
    cfg_path = path + "/config.json";
  } else if (path.size() >= 5 && path.compare(path.size() - 5, 5, ".json") == 0) {
    const size_t slash = path.find_last_of('/');
    *resolved = slash == std::string::npos ? "." : path.substr(0, slash);
    cfg_path = path;
  } else {
    *container = "gguf";
    *resolved = path;
    GGUFFile f;
    f.open(path);
    const GGUFValue* v = f.meta("general.architecture");
    return (v && v->kind == GGUFValue::STRING) ? v->s : std::string("llama");
  }
  *container = "folder";
  std::ifstream in(cfg_path);
  if (!in) throw std::runtime_error("cannot open " + cfg_path);
  std::stringstream ss;
  ss << in.rdbuf();
  const Json cfg = Json::parse(ss.str());
  const Json* a = cfg.find("architecture");
  if (!a || a->kind != Json::STRING) throw std::runtime_error(cfg_path + " names no architecture");
  return a->str;
}

}  // namespace tlhost
