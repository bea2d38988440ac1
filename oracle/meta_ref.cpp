// TEST INFRASTRUCTURE ONLY: the engine sidecar through the reference's own JSON library.
//
// The reference reads and writes "<engine>.meta" with nlohmann::json
// (source/trt_engine/trt_common/trt_meta_data.cpp:49-97), vendored as source under
// source/third_party/json.  trt_meta_data.cpp itself cannot be compiled here (its header pulls
// in NvInfer.h), so this program restates its two functions call for call on top of the real
// library, which is what fixes the text form (std::setw(4) << json) and the reading rules
// (value.get<int>(), iteration over an array or over null).  Built by `make -C oracle ref`
// into oracle/_ref/ when the reference tree is present; the tests use it to check the product's
// reader and writer and to make the committed fixtures under tests/golden/meta/.
//
//   meta_ref write FILE MODE OPT MAX "u0,u1,.." "o0,o1,.." PATH   SaveMetaData of those members
//   meta_ref read FILE      LoadMetaData; prints "ok MODE OPT MAX [u..] [o..] PATH" or "fail"
#include <fstream>
#include <iomanip>
#include <iostream>
#include <nlohmann/json.hpp>
#include <set>
#include <sstream>
#include <string>
#include <vector>

using json = nlohmann::json;

static std::vector<int> ints(const std::string& s) {
  std::vector<int> v;
  std::stringstream ss(s);
  std::string item;
  while (std::getline(ss, item, ','))
    if (!item.empty()) v.push_back(std::stoi(item));
  return v;
}

int main(int argc, char** argv) {
  const std::string cmd = argc > 1 ? argv[1] : "";
  if (cmd == "write" && argc == 9) {
    // trt_meta_data.cpp:81-97
    json meta_json;
    const std::vector<int> u = ints(argv[6]);
    meta_json["infer_mode"] = std::stoi(argv[3]);
    meta_json["opt_batch_size"] = std::stoi(argv[4]);
    meta_json["max_batch_size"] = std::stoi(argv[5]);
    meta_json["unused_input_indices"] = std::set<int>(u.begin(), u.end());
    meta_json["output_indices"] = ints(argv[7]);
    meta_json["torch_module_path"] = std::string(argv[8]);
    std::ofstream meta(argv[2]);
    if (!meta.is_open()) return 2;
    meta << std::setw(4) << meta_json << std::endl;
    return 0;
  }
  if (cmd == "read" && argc == 3) {
    // trt_meta_data.cpp:49-79
    json meta_json;
    std::ifstream meta(argv[2]);
    if (!meta.is_open()) {
      std::cout << "fail" << std::endl;
      return 0;
    }
    try {
      meta >> meta_json;
      const int mode = meta_json["infer_mode"].get<int>();
      const int opt = meta_json["opt_batch_size"].get<int>();
      const int max = meta_json["max_batch_size"].get<int>();
      std::set<int> unused(meta_json["unused_input_indices"].begin(), meta_json["unused_input_indices"].end());
      std::vector<int> out(meta_json["output_indices"].begin(), meta_json["output_indices"].end());
      const std::string path = meta_json["torch_module_path"].get<std::string>();
      std::cout << "ok " << mode << " " << opt << " " << max << " [";
      for (int v : unused) std::cout << v << ",";
      std::cout << "] [";
      for (int v : out) std::cout << v << ",";
      std::cout << "] " << path << std::endl;
    } catch (const std::exception&) {
      std::cout << "fail" << std::endl;
    }
    return 0;
  }
  std::cerr << "usage: meta_ref write FILE MODE OPT MAX UNUSED OUTPUTS PATH | meta_ref read FILE" << std::endl;
  return 2;
}
