// torch.classes.recis.{WriteBlock, Saver, Loader, CheckpointReader}: table checkpoints in the
// reference's directory layout (csrc/serialize/*, registered at csrc/bind.cc:147-170).
//
// A checkpoint directory holds (csrc/serialize/name.cc:15-62, save_bundle.cc:56-330):
//  * model-XXXXXX-of-YYYYYY.safetensors data files, XXXXXX = shard_index * parallel + writer,
//    YYYYYY = parallel * shard_num. Each file is `u64 header_size | header | raw blocks`; the header
//    is compact JSON {name: {"dtype", "shape", "data_offsets"}} in block order, padded with 1..8
//    spaces to a multiple of 8 (table_writer.cc:60-82), offsets relative to the end of the header;
//  * index: {"block_index": {block name: file number}, "file_index": {file name: number}}
//    (index_info.cc:18-27,93-105);
//  * tensorkey.json: on-disk name -> model block name for table blocks (save_bundle.cc:84-105);
//  * torch_rank_weights_embs_table_multi_shard.json: a description of every block for downstream
//    tools (save_bundle.cc:277-318).
// Names. A table block is <child>@<slot> (slot "id" for the keys) with the slice string
// begin@end@size (zero padded to the width of size, slice_info.cc:38-48); its model block name is
// <child>@<slot>^<slice> and its on-disk name <child>.<slot>/part_<shard>_<shards>. A dense tensor
// keeps its name with the slice " ".
//
// Device side of a table block: the key -> row snapshot is split by child on the GPU, the keys go
// to the host once, and every slot is gathered RECIS_BLOCK_WRITE_SIZE rows at a time into one of
// two pinned host buffers, so the copy of one piece overlaps the file write of the piece before.
#pragma once

#include <ATen/ATen.h>
#include <ATen/core/Dict.h>
#include <torch/custom_class.h>

#include <cstdio>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "table.h"

namespace recis {
namespace serialize {

// ---- a small JSON value: objects keep the order of insertion
struct Json {
  enum Kind { kNull, kBool, kInt, kDouble, kString, kArray, kObject };
  Kind kind = kNull;
  bool b = false;
  int64_t i = 0;
  double d = 0;
  std::string s;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;

  static Json Bool(bool v);
  static Json Int(int64_t v);
  static Json Str(std::string v);
  static Json Array();
  static Json Object();
  Json& Set(const std::string& key, Json v);       // replaces or appends
  const Json* Find(const std::string& key) const;  // nullptr when absent
  bool Erase(const std::string& key);
  void SortKeys(bool deep);
  std::string Dump(int indent = -1) const;  // -1: compact (",", ":"), else nlohmann's / Python's indented form
  static Json Parse(const std::string& text);
};

std::string DtypeToString(at::ScalarType dtype);      // dtype_serialize.cc:4-66
at::ScalarType StringToDtype(const std::string& s);
std::string SliceToString(int64_t begin, int64_t end, int64_t size);
std::vector<int64_t> SliceFromString(const std::string& msg);
bool SlicesIntersect(const std::vector<int64_t>& a, const std::vector<int64_t>& b);
std::string DataFileName(int64_t file_index, int64_t file_count);
std::string BlockName(const std::string& tensor_name, const std::string& slice_info);
int64_t BlockWriteSize();  // RECIS_BLOCK_WRITE_SIZE, name.cc:135-142
int64_t BlockReadSize();   // RECIS_BLOCK_READ_SIZE, name.cc:144-151

// One named block of a data file (csrc/serialize/write_block.h:19-44).
class WriteBlock : public torch::CustomClassHolder {
 public:
  WriteBlock(std::string tensor_name, std::string slice_info, bool dense, at::ScalarType dtype,
             std::vector<int64_t> shape);
  ~WriteBlock() override = default;
  const std::string& TensorName() const { return tensor_name_; }
  const std::string& SliceInfo() const { return slice_info_; }
  bool IsDense() const { return dense_; }
  at::ScalarType Dtype() const { return dtype_; }
  const std::vector<int64_t>& Shape() const { return shape_; }
  int64_t NumBytes() const { return nbytes_; }
  void SetTensorName(const std::string& name) { tensor_name_ = name; }
  // write_block.cc:117-121: a renamed table block carries no slice suffix
  std::string MetaKey() const;
  // Writes the block's bytes; returns how many.
  virtual int64_t WriteData(std::FILE* file) = 0;

 protected:
  std::string tensor_name_, slice_info_;
  bool dense_;
  at::ScalarType dtype_;
  std::vector<int64_t> shape_;
  int64_t nbytes_;
};
using WriteBlockPtr = c10::intrusive_ptr<WriteBlock>;

// A dense tensor, copied to the host when the block is made (write_block.cc:88-97).
WriteBlockPtr MakeTensorWriteBlock(const std::string& name, const at::Tensor& tensor);
// A table block whose rows are already in host memory (the keys; also for tools and tests).
WriteBlockPtr MakeArrayWriteBlock(const std::string& name, const std::string& slice_info, const at::Tensor& rows);
// write_block.cc:33-77: per child, the key block then one block per slot, rows in snapshot order.
// Keys of a coalesced table are split by their 12-bit tag and stored without it.
std::vector<WriteBlockPtr> MakeHTWriteBlocks(const HashTablePtr& table);

// table_writer.cc:48-88: header (offsets in block order), then the blocks; json_path gets the header
// with the "dense" flags, for the merge of the side files.
void WriteDataFile(const std::string& path, const std::string& json_path, const std::vector<WriteBlockPtr>& blocks);

// save_bundle.cc:56-330. Blocks go to `parallel` data files round robin in the order they are added;
// every file is written by its own thread. Shard 0 merges the per-shard side files; it waits (up to
// merge_timeout seconds) for those of the other shards.
class SaveBundle : public torch::CustomClassHolder {
 public:
  SaveBundle(std::string path, int64_t parallel, int64_t shard_index, int64_t shard_num, double merge_timeout = 3600.0);
  void AddBlock(const WriteBlockPtr& block);
  void Save();
  void MergeMetaInfo();

 private:
  std::string Tmp(const char* kind, int64_t writer, int64_t shard) const;
  void MergeRankJson();
  void MergeTensorKeyJson();
  std::string path_;
  int64_t parallel_, shard_index_, shard_num_;
  double merge_timeout_;
  std::vector<std::vector<WriteBlockPtr>> writers_;
  std::vector<std::string> file_names_;
  int64_t next_ = 0;
  std::vector<std::pair<std::string, int64_t>> file_index_, block_index_;  // in order of insertion
  std::vector<std::pair<std::string, std::string>> name_map_;
};

struct BlockInfo {
  at::ScalarType dtype;
  std::vector<int64_t> shape;
  int64_t offset_beg = 0, offset_end = 0;  // absolute file offsets
  std::string path;
  int64_t Size() const { return offset_end - offset_beg; }
  int64_t RowBytes() const { return shape.empty() || shape[0] == 0 ? 0 : Size() / shape[0]; }
  void ReadInto(void* out, int64_t byte_offset, int64_t nbytes) const;
  at::Tensor ReadTensor() const;
};

// table_reader.cc:34-60: block name -> BlockInfo with absolute file offsets (names mapped through
// name_map when given), in file order.
std::vector<std::pair<std::string, BlockInfo>> ReadDataFileHeader(const std::string& path,
                                                                  const std::map<std::string, std::string>* name_map);

// load_bundle.cc:17-112: the index and name map of a checkpoint directory; file headers are parsed on
// first use.
class LoadBundle : public torch::CustomClassHolder {
 public:
  explicit LoadBundle(const std::string& path);
  bool HasTensor(const std::string& tensor_name) const;
  std::vector<std::string> ListTensor() const;
  std::vector<std::string> SliceInfos(const std::string& tensor_name) const;
  const BlockInfo& GetBlockInfo(const std::string& block_name);
  std::vector<int64_t> TensorShape(const std::string& tensor_name);
  at::ScalarType TensorType(const std::string& tensor_name);

 private:
  std::string path_;
  std::map<std::string, std::string> name_map_;
  std::vector<std::pair<std::string, int64_t>> block_index_;
  std::map<int64_t, std::string> file_by_number_;
  std::map<int64_t, std::map<std::string, BlockInfo>> headers_;
};

// csrc/serialize/saver.h:10-25
class Saver : public torch::CustomClassHolder {
 public:
  Saver(int64_t shard_index, int64_t shard_num, int64_t parallel, const std::string& path);
  std::vector<WriteBlockPtr> MakeWriteBlocks(const c10::Dict<std::string, HashTablePtr>& hashtables,
                                             const c10::Dict<std::string, at::Tensor>& tensors);
  void Save(std::vector<WriteBlockPtr> write_blocks);

 private:
  int64_t parallel_, shard_index_, shard_num_;
  std::string path_;
};

// csrc/serialize/loader.h:14-36
class Loader : public torch::CustomClassHolder {
 public:
  Loader(const std::string& path, int64_t parallel, c10::Dict<std::string, HashTablePtr> hts_to_load,
         c10::Dict<std::string, at::Tensor> tensors_to_load);
  // {"dst_tensor_name": {"src_tensor_name": ["id", "embedding", ...]}} for tables, an empty slot list
  // for dense tensors (load_info.cc:17-33)
  std::string DefaultLoadInfo();
  void Load(std::string load_info);

 private:
  int64_t parallel_;
  std::string path_;
  std::vector<std::pair<std::string, HashTablePtr>> hts_;
  std::vector<std::pair<std::string, at::Tensor>> tensors_;
};

// csrc/serialize/checkpoint_reader.h:12-27: whole tensors (table blocks of all shards concatenated
// in slice order) into host memory.
class CheckpointReader : public torch::CustomClassHolder {
 public:
  explicit CheckpointReader(const std::string& path) : path_(path) {}
  void Init();
  std::vector<std::string> ListTensors();
  at::Tensor LoadTensor(const std::string& tensor_name);
  std::vector<int64_t> TensorShape(const std::string& tensor_name);
  at::Tensor TensorType(const std::string& tensor_name);  // an empty tensor of the stored dtype

 private:
  LoadBundle& Bundle();
  std::string path_;
  c10::intrusive_ptr<LoadBundle> bundle_;
};

}  // namespace serialize
}  // namespace recis
