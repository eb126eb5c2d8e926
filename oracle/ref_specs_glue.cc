// Test infrastructure, not product code: C entry points over the REFERENCE's own table-spec
// objects (src/storage/specs.cc + include/storage/specs.h + include/common/dtypes.h), compiled
// from where those sources lie by `make -C oracle ref`, so that the CPU tests can compare the
// oracle's and the library's layout arithmetic with the reference's object code.
// Only tests may load the result (oracle/_ref/libref_specs.so).
#include <cstdint>
#include <string>
#include <vector>

#include "common/dtypes.h"
#include "storage/specs.h"

using gear::common::DataType;
using gear::storage::ColumnSpec;
using gear::storage::TableSpec;

namespace {
std::vector<ColumnSpec> columns(int ncols, const int64_t *shapes, const int *ndims,
                                const int *dtypes) {
  std::vector<ColumnSpec> cols;
  const int64_t *s = shapes;
  for (int c = 0; c < ncols; ++c) {
    std::vector<size_t> shape(s, s + ndims[c]);
    s += ndims[c];
    cols.emplace_back(shape, static_cast<DataType>(dtypes[c]), "col" + std::to_string(c));
  }
  return cols;
}
}  // namespace

extern "C" {

// sizeof_dtype (include/common/dtypes.h:55-76); -1 where the reference throws
__attribute__((visibility("default"))) int64_t ref_sizeof_dtype(int dtype) {
  try {
    return (int64_t)gear::common::sizeof_dtype(static_cast<DataType>(dtype));
  } catch (const std::exception &) {
    return -1;
  }
}

// ColumnSpec::size (src/storage/specs.cc:10-14)
__attribute__((visibility("default"))) int64_t ref_column_size(const int64_t *shape, int ndim,
                                                               int dtype) {
  try {
    std::vector<size_t> s(shape, shape + ndim);
    return (int64_t)ColumnSpec(s, static_cast<DataType>(dtype)).size();
  } catch (const std::exception &) {
    return -1;
  }
}

// TableSpec::TableSpec / size (src/storage/specs.cc:16-29, 42)
__attribute__((visibility("default"))) int64_t ref_table_nbytes(int64_t trajectory_length,
                                                                int64_t capacity, int ncols,
                                                                const int64_t *shapes,
                                                                const int *ndims,
                                                                const int *dtypes) {
  try {
    TableSpec t(0, 1, (size_t)trajectory_length, (size_t)capacity, (size_t)ncols,
                columns(ncols, shapes, ndims, dtypes));
    return (int64_t)t.size();
  } catch (const std::exception &) {
    return -1;
  }
}

// TableSpec::index (src/storage/specs.cc:31-40) over columns named col0, col1, ...
__attribute__((visibility("default"))) int64_t ref_table_index(int ncols, const int64_t *shapes,
                                                               const int *ndims, const int *dtypes,
                                                               const char *name) {
  TableSpec t(0, 1, 1, 1, (size_t)ncols, columns(ncols, shapes, ndims, dtypes));
  return (int64_t)t.index(name);
}
}
