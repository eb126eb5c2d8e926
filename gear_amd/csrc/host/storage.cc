#include "storage.hpp"

#include <numeric>
#include <sstream>
#include <stdexcept>

namespace gearhost {

size_t ColumnSpec::size() const {
  size_t n = sizeof_dtype(dtype);
  for (size_t d : shape) n *= d;
  return n;
}

TableSpec::TableSpec(size_t rank, size_t worldsize, size_t trajectory_length, size_t capacity,
                     size_t num_columns, std::vector<ColumnSpec> column_specs)
    : rank(rank), worldsize(worldsize), trajectory_length(trajectory_length), capacity(capacity),
      num_columns(num_columns), column_specs(std::move(column_specs)) {
  if (this->column_specs.size() != num_columns) {
    std::stringstream ss;
    ss << "column specs size mismatch with declared number of columns: spec num "
       << this->column_specs.size() << ", expected " << num_columns;
    throw std::runtime_error(ss.str());
  }
  size_t total = 0;
  for (const ColumnSpec &c : this->column_specs) total += c.size();
  nbytes = total * trajectory_length * capacity;
}

ssize_t TableSpec::index(const std::string &name) const {
  for (size_t i = 0; i < column_specs.size(); ++i)
    if (column_specs[i].name == name) return (ssize_t)i;
  return -1;
}

TrajectoryTable::TrajectoryTable(const TableSpec &spec, key_t key, bool create, Placement placement)
    : spec_(spec) {
  size_t sum = 0;
  accu_strides_.push_back(0);
  for (const ColumnSpec &c : spec_.column_specs) {
    column_strides_.push_back(c.size());
    sum += c.size();
    accu_strides_.push_back(sum);
  }
  trajectory_stride_ = sum * spec_.trajectory_length;
  block_ = std::make_unique<MemoryBlock>(trajectory_stride_ * spec_.capacity, placement, key, create);
}

const ColumnSpec &TrajectoryTable::column_spec(size_t c) const {
  if (c >= spec_.column_specs.size()) throw std::out_of_range("column id out of range");
  return spec_.column_specs[c];
}

std::string SubscribePattern::to_string() const {
  const char *p = pad_option == PadOption::kInactive ? "PadOption::kInactive"
                  : pad_option == PadOption::kHead   ? "PadOption::kHead"
                  : pad_option == PadOption::kTail   ? "PadOption::kTail"
                                                     : "PadOption: kUnknown";
  std::stringstream ss;
  ss << "<SubscribePattern: offset " << offset << ", length " << length << ", " << p << ">";
  return ss.str();
}

StorageHandler::StorageHandler(std::shared_ptr<TrajectoryTable> table, size_t global_capacity,
                               Range wregion, Range rregion)
    : table_(std::move(table)), global_capacity_(global_capacity), wregion_(wregion),
      rregion_(rregion) {
  patterns_.resize(table_->ncolumns());
}

void StorageHandler::set(const std::vector<size_t> &cids,
                         const std::vector<SubscribePattern> &patterns) {
  if (patterns.size() < cids.size())
    throw std::runtime_error("fewer SubscribePatterns than column ids");
  for (size_t k = 0; k < cids.size(); ++k) {
    if (cids[k] >= patterns_.size()) throw std::runtime_error("column id out of range");
    patterns_[cids[k]] = patterns[k];
  }
}

ColumnWindow StorageHandler::window(size_t column) const {
  if (column >= patterns_.size() || !patterns_[column].has_value())
    throw std::runtime_error("Subscribing a column without setting its SubscribePattern.");
  const SubscribePattern &p = *patterns_[column];
  ColumnWindow w;
  w.ofst = p.offset;
  w.span = (int64_t)p.length;
  w.step_bytes = (int64_t)table_->column_stride(column);
  w.col_base = (int64_t)table_->column_base(column);
  w.dst_stride = w.span * w.step_bytes;
  w.pad_head = p.pad_option == SubscribePattern::PadOption::kHead;
  return w;
}

int64_t StorageHandler::sub(int64_t num, const int64_t *idxs, const int64_t *tss,
                            const int64_t *lens, size_t column, int64_t *src_offsets,
                            int64_t *dst_offsets, int64_t *copy_lens) const {
  const ColumnWindow w = window(column);
  const int64_t traj_stride = (int64_t)table_->trajectory_stride();
  for (int64_t i = 0; i < num; ++i) {
    int64_t first = tss[i] + w.ofst;  // first step of the window, clamped into the trajectory
    if (first < 0) first = 0;
    int64_t last = first + w.span;  // one past the last step, clamped to the trajectory length
    if (last > lens[i]) last = lens[i];
    int64_t bytes = (last - first) * w.step_bytes;
    if (bytes < 0) bytes = 0;
    copy_lens[i] = bytes;
    src_offsets[i] = idxs[i] * traj_stride + w.col_base + first * w.step_bytes;
    dst_offsets[i] = i * w.dst_stride + (w.pad_head ? w.dst_stride - bytes : 0);
  }
  return w.dst_stride;
}

void StorageHandler::view_range(size_t index, size_t column, size_t *offset, size_t *length) const {
  if (column >= table_->ncolumns()) throw std::out_of_range("column id out of range");
  *offset = index * table_->trajectory_stride() + table_->column_base(column);
  *length = table_->column_stride(column) * table_->table_spec().trajectory_length;
}

const void *StorageHandler::device_base() const {
  const MemoryBlock &b = table_->block();
  if (b.device() != nullptr) return b.device();
  if (b.any() == nullptr) throw std::runtime_error("table memory is not connected (call connect())");
  throw std::runtime_error(
      std::string("table memory (") + placement_name(b.placement()) +
      ") is not visible to the GPU: create the table with placement 'pinned' or 'device', or set "
      "GEAR_HIP_HOST_REGISTER=1 where the ROCm host allows pinning shared memory");
}

}  // namespace gearhost
