// Table specs, byte layout, window patterns and the storage handler (host side of the gather).
//
// Layout of a table (reference src/storage/table.cc:8-25, src/storage/handler.cc:93-96,223-229):
//   step bytes of column c      s_c = sizeof(dtype_c) * prod(shape_c)
//   byte address of (i, c, t) = i * S + A_c * T + t * s_c,   A_c = sum_{j<c} s_j,  S = T * sum s_c
// i.e. [trajectory][column][timestep][element bytes], no padding anywhere.
#pragma once
#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "dtypes.hpp"
#include "memory.hpp"

namespace gearhost {

struct ColumnSpec {
  std::vector<size_t> shape;
  DataType dtype;
  std::string name;
  ColumnSpec(std::vector<size_t> shape, DataType dtype, std::string name = "")
      : shape(std::move(shape)), dtype(dtype), name(std::move(name)) {}
  size_t size() const;  // bytes per step
};

struct TableSpec {
  size_t rank, worldsize, trajectory_length, capacity, num_columns;
  std::vector<ColumnSpec> column_specs;
  size_t nbytes;
  TableSpec(size_t rank, size_t worldsize, size_t trajectory_length, size_t capacity,
            size_t num_columns, std::vector<ColumnSpec> column_specs);
  ssize_t index(const std::string &name) const;  // -1 when absent
  size_t size() const { return nbytes; }
};

class TrajectoryTable {
 public:
  TrajectoryTable(const TableSpec &spec, key_t key, bool create, Placement placement);
  ssize_t connect() { return block_->alloc(); }
  size_t ncolumns() const { return spec_.num_columns; }
  const TableSpec &table_spec() const { return spec_; }
  const ColumnSpec &column_spec(size_t c) const;
  MemoryBlock &block() const { return *block_; }
  size_t trajectory_stride() const { return trajectory_stride_; }
  size_t column_stride(size_t c) const { return column_strides_.at(c); }
  size_t accu_stride(size_t c) const { return accu_strides_.at(c); }
  size_t column_base(size_t c) const { return accu_strides_.at(c) * spec_.trajectory_length; }

 private:
  TableSpec spec_;
  std::unique_ptr<MemoryBlock> block_;
  size_t trajectory_stride_;
  std::vector<size_t> column_strides_, accu_strides_;
};

struct SubscribePattern {
  enum class PadOption : int { kInactive = 0, kHead = 1, kTail = 2, kUnknown = 3 };
  int offset;
  size_t length;
  PadOption pad_option;
  SubscribePattern(int offset, size_t length, PadOption opt = PadOption::kTail)
      : offset(offset), length(length), pad_option(opt) {}
  std::string to_string() const;
};

struct Range {
  size_t lb, hb;
  Range(size_t lb, size_t hb) : lb(lb), hb(hb) {}
};

// Arguments of one column for the device gather, derived from table + pattern.
struct ColumnWindow {
  int64_t ofst, span, step_bytes, col_base, dst_stride;
  bool pad_head;
};

class StorageHandler {
 public:
  StorageHandler(std::shared_ptr<TrajectoryTable> table, size_t global_capacity, Range wregion,
                 Range rregion);
  void set(const std::vector<size_t> &cids, const std::vector<SubscribePattern> &patterns);
  // handler.cc:78-131; arrays are host memory of `num` entries each; returns length * s_c
  int64_t sub(int64_t num, const int64_t *idxs, const int64_t *tss, const int64_t *lens,
              size_t column, int64_t *src_offsets, int64_t *dst_offsets, int64_t *copy_lens) const;
  ColumnWindow window(size_t column) const;  // throws when the column has no pattern
  const TrajectoryTable &table() const { return *table_; }
  // byte range of (trajectory index, column): handler.cc:223-234
  void view_range(size_t index, size_t column, size_t *offset, size_t *length) const;
  // the address the GPU gathers from; throws when the table is not GPU-visible
  const void *device_base() const;

 private:
  std::shared_ptr<TrajectoryTable> table_;
  size_t global_capacity_;
  Range wregion_, rregion_;
  std::vector<std::optional<SubscribePattern>> patterns_;
};

}  // namespace gearhost
