// TensorFile: the .npz container the reference's tools pass weights, inputs and results in
// (include/tpuc/Support/TensorFile.h:83-319, a map of name -> array kept in memory and
// written back as a whole by keep(); third_party cnpy does the zip / .npy work there).
// Same operations and the same on-disk result here: a zip archive with one `<name>.npy`
// member per array, stored uncompressed (what cnpy writes and numpy.savez writes); members
// compressed with deflate (numpy.savez_compressed) are read through zlib.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace tpuhip {

struct NpyArray {
  std::vector<int64_t> shape;
  char kind = 'f';           // numpy kind: 'f' float, 'i' signed, 'u' unsigned, 'b' bool
  int word_size = 4;         // bytes per element
  bool fortran_order = false;
  std::vector<uint8_t> bytes;
  size_t count() const;                       // product of the shape
  size_t num_bytes() const { return bytes.size(); }
};

class TensorFile {
public:
  // readOnly: the file must exist and hold at least one array (TensorFile.h:85-105);
  // newCreate: start empty whatever is on disk
  TensorFile(const std::string &filename, bool readOnly, bool newCreate = false);

  // addTensor: fails (returns false) if the name is already used (TensorFile.h:139-157)
  bool addTensor(const std::string &name, const float *data, const std::vector<int64_t> &shape);
  bool addTensor(const std::string &name, const NpyArray &array);
  // readTensor<float>(name, data, count): the stored array must be float32 of exactly count
  // elements (TensorFile.h:188-202 compares the byte counts); returns false otherwise
  bool readTensor(const std::string &name, float *data, size_t count) const;
  // any numeric array converted to float, for inputs written by other tools as int8 / uint8 / ...
  bool readTensorAsFloat(const std::string &name, std::vector<float> &data, std::vector<int64_t> &shape) const;
  bool deleteTensor(const std::string &name);
  // readAllTensors (TensorFile.h:236-256): float32 arrays only, in name order
  void readAllTensors(std::vector<std::string> &names, std::vector<std::vector<float>> &tensors,
                      std::vector<std::vector<int64_t>> &shapes) const;
  const NpyArray *find(const std::string &name) const;
  std::vector<std::string> names() const;
  // keep(): writes the whole map to the file if anything was added or deleted; returns the
  // number of changes written (TensorFile.h:258-296, without the rename-on-increment option)
  int keep();
  const std::string &path() const { return filename; }

private:
  void load();
  std::string filename;
  bool readOnly;
  std::map<std::string, NpyArray> map;
  int changes = 0;
};

std::unique_ptr<TensorFile> openInputTensorFile(const std::string &filename);
std::unique_ptr<TensorFile> openOutputTensorFile(const std::string &filename);

}  // namespace tpuhip
