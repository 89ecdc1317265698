// Option table of the engine and a reader for the flat JSON file the Python
// wrapper hands to init().  Field names, types and defaults are those of the
// reference's ConfigProto (cuhnsw/proto/config.proto:10-26); parsing replaces the
// reference's json11 use in CuHNSW::Init (cpp/src/cuhnsw_base.cu:67-106).
#pragma once
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <map>
#include <sstream>
#include <string>

namespace cuhnsw_amd {

enum DistType { DIST_DOT = 0, DIST_L2 = 1 };

struct Options {
  int seed = 777;
  int c_log_level = 2;
  int py_log_level = 2;
  int max_m = 12;
  int max_m0 = 24;
  int ef_construction = 150;
  double level_mult = 0.0;
  bool save_remains = false;
  double hyper_threads = 10.0;
  int block_dim = 32;
  std::string dist_type = "dot";
  int visited_table_size = 0;
  int visited_list_size = 8192;
  bool nrz = false;
  bool reverse_cand = false;
  double heuristic_coef = 0.25;
};

// Minimal reader for one flat JSON object whose values are numbers, strings,
// true/false/null.  Returns false on malformed input.
inline bool parse_flat_json(const std::string& text, std::map<std::string, std::string>& out) {
  size_t i = 0;
  const size_t n = text.size();
  auto skip = [&]() { while (i < n && std::isspace((unsigned char)text[i])) ++i; };
  auto read_string = [&](std::string& s) -> bool {
    if (i >= n || text[i] != '"') return false;
    ++i;
    s.clear();
    while (i < n && text[i] != '"') {
      if (text[i] == '\\' && i + 1 < n) ++i;
      s.push_back(text[i++]);
    }
    if (i >= n) return false;
    ++i;
    return true;
  };
  skip();
  if (i >= n || text[i] != '{') return false;
  ++i;
  skip();
  if (i < n && text[i] == '}') return true;
  while (i < n) {
    skip();
    std::string key, val;
    if (!read_string(key)) return false;
    skip();
    if (i >= n || text[i] != ':') return false;
    ++i;
    skip();
    if (i < n && text[i] == '"') {
      if (!read_string(val)) return false;
    } else {
      while (i < n && text[i] != ',' && text[i] != '}' && !std::isspace((unsigned char)text[i])) val.push_back(text[i++]);
      if (val.empty()) return false;
    }
    out[key] = val;
    skip();
    if (i < n && text[i] == ',') { ++i; continue; }
    if (i < n && text[i] == '}') return true;
    return false;
  }
  return false;
}

// 0 ok, 1 unreadable / malformed / out of range, 2 invalid dist_type; `why` receives the reason of a failure
inline int load_options(const std::string& path, Options& o, int& dist_type, std::string& why) {
  std::ifstream f(path);
  if (!f.is_open()) {
    why = "cannot read option file: " + path;
    return 1;
  }
  std::stringstream ss;
  ss << f.rdbuf();
  std::map<std::string, std::string> kv;
  if (!parse_flat_json(ss.str(), kv)) {
    why = "cannot parse option file: " + path;
    return 1;
  }
  auto num = [&](const char* k, double def) {
    auto it = kv.find(k);
    if (it == kv.end() || it->second == "null") return def;
    if (it->second == "true") return 1.0;
    if (it->second == "false") return 0.0;
    return std::atof(it->second.c_str());
  };
  o.seed = (int)num("seed", o.seed);
  o.c_log_level = (int)num("c_log_level", o.c_log_level);
  o.py_log_level = (int)num("py_log_level", o.py_log_level);
  o.max_m = (int)num("max_m", o.max_m);
  o.max_m0 = (int)num("max_m0", o.max_m0);
  o.ef_construction = (int)num("ef_construction", o.ef_construction);
  o.level_mult = num("level_mult", o.level_mult);
  o.save_remains = num("save_remains", o.save_remains) != 0.0;
  o.hyper_threads = num("hyper_threads", o.hyper_threads);
  o.block_dim = (int)num("block_dim", o.block_dim);
  o.visited_table_size = (int)num("visited_table_size", o.visited_table_size);
  o.visited_list_size = (int)num("visited_list_size", o.visited_list_size);
  o.nrz = num("nrz", o.nrz) != 0.0;
  o.reverse_cand = num("reverse_cand", o.reverse_cand) != 0.0;
  o.heuristic_coef = num("heuristic_coef", o.heuristic_coef);
  auto it = kv.find("dist_type");
  if (it != kv.end()) o.dist_type = it->second;
  if (o.dist_type == "dot") dist_type = DIST_DOT;
  else if (o.dist_type == "l2") dist_type = DIST_L2;
  else {
    why = "invalid dist type " + o.dist_type;
    return 2;
  }
  // the index file keeps a link count in 16 bits
  if (o.max_m < 1 || o.max_m0 < 1 || o.max_m > 65535 || o.max_m0 > 65535) {
    why = "max_m and max_m0 must lie in 1..65535";
    return 1;
  }
  if (o.ef_construction < 1) {
    why = "ef_construction must be positive";
    return 1;
  }
  return 0;
}

}  // namespace cuhnsw_amd
