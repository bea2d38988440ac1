// The engine sidecar ("<engine file>.meta"): the settings an engine file needs beside its
// plugins, typed.  Twin of EngineMetaData (source/trt_engine/trt_common/trt_meta_data.h:37-90):
// same members, same defaults, same JSON keys and value types, same text form on disk
// (source/trt_engine/trt_common/trt_meta_data.cpp:42-97), so a sidecar written here loads in the
// reference and the other way round.  Host code only.
#pragma once

#include <set>
#include <string>
#include <vector>

namespace fwdmi {

// InferMode, source/common/fwd_common.h:40-46
enum class InferMode : int { FLOAT = 0, HALF = 1, INT8 = 2, INT8_CALIB = 3, INVALID = -1 };

class EngineMetaData {
 public:
  InferMode Mode() const { return mode_; }
  void SetMode(InferMode mode) { mode_ = mode; }
  int MaxBatchSize() const { return max_batch_size_; }
  void SetMaxBatchSize(int v) { max_batch_size_ = v; }
  int OptBatchSize() const { return opt_batch_size_; }
  void SetOptBatchSize(int v) { opt_batch_size_ = v; }
  const std::set<int>& UnusedInputIndices() const { return unused_input_indices_; }
  void SetUnusedInputIndices(const std::set<int>& v) { unused_input_indices_ = v; }
  const std::vector<int>& OutputPositions() const { return output_pos_; }
  void SetOutputPositions(const std::vector<int>& v) { output_pos_ = v; }
  const std::string& TorchModulePath() const { return torch_module_path_; }
  void SetTorchModulePath(const std::string& path) { torch_module_path_ = path; }

  // Reads the sidecar.  False (with the reason recorded as the thread's last error) when the file
  // cannot be opened, is not JSON, lacks infer_mode / opt_batch_size / max_batch_size /
  // torch_module_path, or holds a value of the wrong type.  The two index arrays may be absent
  // (the reference reads an absent array as empty); unknown keys are ignored.
  bool LoadMetaData(const std::string& meta_file);
  // The same from text.
  bool ParseMetaData(const std::string& json_text);
  // Writes the sidecar in the reference's form: keys in alphabetical order, four-space
  // indentation, one array element per line, a trailing newline.
  bool SaveMetaData(const std::string& meta_file) const;
  std::string ToJson() const;

 private:
  InferMode mode_{InferMode::FLOAT};
  int max_batch_size_{-1};
  int opt_batch_size_{-1};
  std::string torch_module_path_;
  std::set<int> unused_input_indices_;  // inputs of the traced module the engine does not bind
  std::vector<int> output_pos_;         // engine binding index of every output, in the module's order
};

}  // namespace fwdmi
