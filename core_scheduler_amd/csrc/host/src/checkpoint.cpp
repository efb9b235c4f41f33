// cs::save / cs::load: checkpoints in the reference's file format
// (the reference's src/module/module.cpp:129-220).
//
// One Parquet file with two columns, `key: string` (the qualified parameter name, e.g.
// "h.0.ln_1.weight") and `value: list<item: float>` (the parameter flattened and widened to
// float32), one row per parameter, a single row group.  load looks every key of the file up in
// named_parameters() (an unknown key aborts, as in the reference) and copies the values,
// converted to the parameter's dtype and device and viewed in its shape, into the parameter.
//
// The reference leaves optimizer checkpoints unimplemented
// (src/module/optimizer_module.cpp:45-51: both functions abort).  Here they write AdamW's
// first and second moments (and v_max) in the same layout under "<parameter>.m", ".v",
// ".v_max", plus one row "<parameter>.t" with the step count as two floats (t mod 2^24,
// t div 2^24: both exact in float32), so that a run resumes with the state it stopped with.
//
// Host-side file work; the only device work is the copies to and from the host.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/ops/from_blob.h>
#include <arrow/api.h>
#include <arrow/io/file.h>
#include <parquet/arrow/reader.h>
#include <parquet/arrow/writer.h>

#include <cmath>
#include <string>
#include <utility>
#include <vector>

#include "logger.h"
#include "module/module.h"
#include "module/optimizer_module.h"
#include "optimizer/adamw.h"
#include "tensor_impl.h"

namespace cs {
namespace {
constexpr long kTSplit = 1L << 24;  // floats hold every integer up to here

using Rows = std::vector<std::pair<std::string, at::Tensor>>;  // name, flat float32 CPU tensor

at::Tensor to_host_floats(const ReadOnlyTensor &t, const std::string &name) {
  t.wait();
  const at::Tensor &src = t.impl()->tensor();
  CS_ASSERT_TRUE(src.defined(), "cannot save " + name + ": it has no value yet");
  return src.detach().cpu().to(at::kFloat).contiguous().view({-1});
}

void write_rows(const Rows &rows, const std::string &path) {
  arrow::MemoryPool *pool = arrow::default_memory_pool();
  const auto schema = arrow::schema(
      {arrow::field("key", arrow::utf8()), arrow::field("value", arrow::list(arrow::field("item", arrow::float32())))});
  arrow::StringBuilder keys(pool);
  arrow::ListBuilder values(pool, std::make_shared<arrow::FloatBuilder>(pool));
  auto *floats = dynamic_cast<arrow::FloatBuilder *>(values.value_builder());
  for (const auto &[name, flat] : rows) {
    CS_ASSERT_TRUE(keys.Append(name).ok(), "Writing failed");
    CS_ASSERT_TRUE(values.Append().ok(), "Writing failed");
    CS_ASSERT_TRUE(floats->AppendValues(flat.data_ptr<float>(), flat.numel()).ok(), "Writing failed");
  }
  std::shared_ptr<arrow::Array> key_array, value_array;
  CS_ASSERT_TRUE(keys.Finish(&key_array).ok(), "Writing failed");
  CS_ASSERT_TRUE(values.Finish(&value_array).ok(), "Writing failed");
  const auto table = arrow::Table::Make(schema, {key_array, value_array});
  auto outfile = arrow::io::FileOutputStream::Open(path);
  CS_ASSERT_TRUE(outfile.ok(), "cannot open " + path + " for writing: " + outfile.status().ToString());
  const int64_t row_group = rows.empty() ? 1 : static_cast<int64_t>(rows.size());  // one row group, as the reference writes
  const auto st = parquet::arrow::WriteTable(*table, pool, *outfile, row_group);
  CS_ASSERT_TRUE(st.ok(), "writing " + path + " failed: " + st.ToString());
  CS_ASSERT_TRUE((*outfile)->Close().ok(), "closing " + path + " failed");
}

Rows read_rows(const std::string &path) {
  arrow::MemoryPool *pool = arrow::default_memory_pool();
  auto infile = arrow::io::ReadableFile::Open(path, pool);
  CS_ASSERT_TRUE(infile.ok(), "Open File failed with error " + infile.status().ToString());
  auto reader = parquet::arrow::OpenFile(*infile, pool);
  CS_ASSERT_TRUE(reader.ok(), "Open File failed with error " + reader.status().ToString());
  const auto read = (*reader)->ReadTable();
  CS_ASSERT_TRUE(read.ok(), "Read File failed with error " + read.status().ToString());
  const std::shared_ptr<arrow::Table> &table = *read;
  CS_ASSERT_TRUE(table->num_columns() == 2 && table->schema()->field(0)->name() == "key" &&
                     table->schema()->field(1)->name() == "value",
                 path + " is not a parameter checkpoint (columns key, value)");
  Rows rows;
  // every chunk (the reference reads chunk 0 only, which is all a file it wrote has)
  for (int c = 0; c < table->column(0)->num_chunks(); ++c) {
    const auto keys = std::dynamic_pointer_cast<arrow::StringArray>(table->column(0)->chunk(c));
    const auto lists = std::dynamic_pointer_cast<arrow::ListArray>(table->column(1)->chunk(c));
    CS_ASSERT_TRUE(keys != nullptr && lists != nullptr, path + ": key must be a string and value a list");
    const auto floats = std::dynamic_pointer_cast<arrow::FloatArray>(lists->values());
    CS_ASSERT_TRUE(floats != nullptr, path + ": value must be a list of float32");
    for (int64_t i = 0; i < keys->length(); ++i) {
      const int64_t off = lists->value_offset(i), len = lists->value_length(i);
      at::Tensor flat = at::empty({len}, at::TensorOptions().dtype(at::kFloat));
      if (len > 0) std::memcpy(flat.data_ptr<float>(), floats->raw_values() + off, sizeof(float) * len);
      rows.emplace_back(keys->GetString(i), std::move(flat));
    }
  }
  return rows;
}

// values -> parameter: converted to its dtype and device, viewed in its shape
void assign(const ReadOnlyTensor &target, const at::Tensor &flat, const std::string &name) {
  target.wait();
  at::Tensor &dst = target.impl()->tensor();
  CS_ASSERT_TRUE(dst.defined(), "cannot load " + name + ": the model's tensor has no value yet");
  CS_ASSERT_TRUE(flat.numel() == dst.numel(), name + ": the file holds " + std::to_string(flat.numel()) +
                                                  " values, the model's tensor " + std::to_string(dst.numel()));
  (void)dst.copy_(flat.to(dst.options()).view(dst.sizes()));
  if (dst.is_cuda()) {
    // the copy ran on the current stream of the tensor's device; tasks on the scheduler's streams
    // that use the parameter next must find it complete
    const c10::hip::HIPGuardMasqueradingAsCUDA guard{dst.device()};
    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().synchronize();
  }
}

std::shared_ptr<optimizer::AdamW::State> adamw_state(const std::shared_ptr<module::OptimizerState> &state,
                                                     const std::string &name) {
  const auto s = std::dynamic_pointer_cast<optimizer::AdamW::State>(state);
  CS_ASSERT_TRUE(s != nullptr, "optimizer checkpoints cover AdamW states; " + name + " is of another kind");
  return s;
}
}  // namespace

void save(const module::Module &module, const std::string &path) {
  Rows rows;
  for (const auto &kv : module.named_parameters()) rows.emplace_back(kv.key(), to_host_floats(kv.value(), kv.key()));
  write_rows(rows, path);
}

void load(const module::Module &module, const std::string &path) {
  const auto parameters = module.named_parameters();
  for (const auto &[key, flat] : read_rows(path)) {
    const auto *found = parameters.find(key);
    CS_ASSERT_TRUE(found != nullptr, "wrong parameter name " + key + " in saved model");
    assign(*found, flat, key);
  }
}

void save(const module::OptimizerModule &module, const std::string &path) {
  Rows rows;
  for (const auto &kv : module.named_states()) {
    const auto s = adamw_state(kv.value(), kv.key());
    rows.emplace_back(kv.key() + ".m", to_host_floats(s->tensors.m, kv.key() + ".m"));
    rows.emplace_back(kv.key() + ".v", to_host_floats(s->tensors.v, kv.key() + ".v"));
    if (s->options.amsgrad) rows.emplace_back(kv.key() + ".v_max", to_host_floats(s->tensors.v_max, kv.key() + ".v_max"));
    at::Tensor t = at::empty({2}, at::TensorOptions().dtype(at::kFloat));
    t.data_ptr<float>()[0] = static_cast<float>(s->options.t % kTSplit);
    t.data_ptr<float>()[1] = static_cast<float>(s->options.t / kTSplit);
    rows.emplace_back(kv.key() + ".t", std::move(t));
  }
  write_rows(rows, path);
}

void load(const module::OptimizerModule &module, const std::string &path) {
  const auto states = module.named_states();
  for (const auto &[key, flat] : read_rows(path)) {
    const auto dot = key.rfind('.');
    CS_ASSERT_TRUE(dot != std::string::npos, "not an optimizer checkpoint row: " + key);
    const std::string name = key.substr(0, dot), field = key.substr(dot + 1);
    const auto *found = states.find(name);
    CS_ASSERT_TRUE(found != nullptr, "wrong parameter name " + name + " in saved optimizer state");
    const auto s = adamw_state(*found, name);
    if (field == "m") {
      assign(s->tensors.m, flat, key);
    } else if (field == "v") {
      assign(s->tensors.v, flat, key);
    } else if (field == "v_max") {
      CS_ASSERT_TRUE(s->options.amsgrad, key + ": this optimizer keeps no v_max (amsgrad is off)");
      assign(s->tensors.v_max, flat, key);
    } else if (field == "t") {
      CS_ASSERT_TRUE(flat.numel() == 1 || flat.numel() == 2, key + ": the step count is one or two values");
      const float *v = flat.data_ptr<float>();
      s->options.t = std::lround(v[0]) + (flat.numel() == 2 ? std::lround(v[1]) * kTSplit : 0L);
    } else {
      CS_ASSERT_TRUE(false, "not an optimizer checkpoint row: " + key);
    }
  }
}
}  // namespace cs
