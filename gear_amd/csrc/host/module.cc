// pybind11 module `_libgear` (imported as gear_amd.libgear): the reference's `libgear.core`
// surface (src/pybind.cc:75-109 and the per-directory pybind.cc files) over the host classes of
// this directory and the C ABI of libgearhip.so.  torch tensors are taken as Python objects
// (data_ptr / numel / ...), so the module does not link libtorch.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstdio>
#include <cstring>
#include <map>
#include <sstream>

#include "gear_hip.h"
#include "indexset.hpp"
#include "requests.hpp"
#include "storage.hpp"

namespace py = pybind11;
using namespace gearhost;

namespace {

void check_hip(const char *what, int rc) {
  if (rc != 0) {
    std::stringstream ss;
    ss << what << " failed: " << gear_hip_error_string(rc) << " (code " << rc << ")";
    throw std::runtime_error(ss.str());
  }
}

py::module_ &torch_module() {
  static py::module_ *torch = new py::module_(py::module_::import("torch"));
  return *torch;
}

struct TensorInfo {
  void *ptr;
  int64_t numel;
  int64_t elem;
  bool cuda;
};

TensorInfo tensor_info(const py::handle &t, const char *name, int64_t want_elem = 0,
                       int need_cuda = -1) {
  if (!py::hasattr(t, "data_ptr") || !py::hasattr(t, "numel"))
    throw py::type_error(std::string(name) + " must be a torch.Tensor");
  if (!t.attr("is_contiguous")().cast<bool>())
    throw std::runtime_error(std::string(name) + " must be contiguous");
  TensorInfo i;
  i.ptr = reinterpret_cast<void *>(t.attr("data_ptr")().cast<uintptr_t>());
  i.numel = t.attr("numel")().cast<int64_t>();
  i.elem = t.attr("element_size")().cast<int64_t>();
  i.cuda = t.attr("is_cuda").cast<bool>();
  if (want_elem && i.elem != want_elem)
    throw std::runtime_error(std::string(name) + " has the wrong element size");
  if (need_cuda == 1 && !i.cuda) throw std::runtime_error(std::string(name) + " must live on the GPU");
  if (need_cuda == 0 && i.cuda) throw std::runtime_error(std::string(name) + " must live on the host");
  return i;
}

// torch._C._cuda_getCurrentRawStream(device) where this torch has it (one C call), else
// torch.cuda.current_stream().cuda_stream
void *current_stream() {
  // the two callables are kept for the life of the process (never destroyed: static py::objects
  // would be released after the interpreter has gone)
  static py::object *raw = nullptr, *getdev = nullptr;
  static bool probed = false;
  if (!probed) {
    probed = true;
    py::object c = torch_module().attr("_C");
    if (py::hasattr(c, "_cuda_getCurrentRawStream") && py::hasattr(c, "_cuda_getDevice")) {
      raw = new py::object(c.attr("_cuda_getCurrentRawStream"));
      getdev = new py::object(c.attr("_cuda_getDevice"));
    }
  }
  if (raw != nullptr) return reinterpret_cast<void *>((*raw)((*getdev)()).cast<uintptr_t>());
  py::object s = torch_module().attr("cuda").attr("current_stream")();
  return reinterpret_cast<void *>(s.attr("cuda_stream").cast<uintptr_t>());
}

// Device scratch owned by the module, one per (purpose, stream), grown on demand and kept (the
// C ABI itself never allocates; calls on different streams must not share a workspace).
void *workspace(const char *tag, void *stream, size_t bytes, size_t *have) {
  static std::map<std::pair<std::string, void *>, std::pair<void *, size_t>> cache;
  auto &e = cache[std::make_pair(std::string(tag), stream)];
  if (e.second < bytes) {
    if (e.first) gear_hip_device_free(e.first);
    e.first = nullptr;
    e.second = 0;
    const size_t want = (bytes + 4095) / 4096 * 4096;
    check_hip("workspace allocation", gear_hip_device_alloc(want, &e.first));
    e.second = want;
  }
  *have = e.second;
  return e.first;
}

// ---- spans: typed (pointer, element count) views, src/common of the reference ------------------
struct SpanBase {
  void *ptr = nullptr;
  int64_t size = 0;  // elements
  bool device = false;
  std::shared_ptr<void> keep;  // whatever owns the memory
};

template <DataType DT>
struct Span : SpanBase {
  Span() = default;
  Span(void *p, int64_t n, bool dev = false, std::shared_ptr<void> k = nullptr) {
    ptr = p;
    size = n;
    device = dev;
    keep = std::move(k);
  }
};

py::object span_to_tensor(const SpanBase &s, int64_t bytes, DataType dt) {
  if (s.device)
    throw std::runtime_error("this span points into a device-resident table; read it with copy_to()");
  const int64_t elem = (int64_t)sizeof_dtype(dt);
  const int64_t n = bytes / elem;
  py::object base = py::none();
  if (s.keep) base = py::capsule(new std::shared_ptr<void>(s.keep), [](void *p) {
      delete static_cast<std::shared_ptr<void> *>(p);
    });
  else
    base = py::capsule(s.ptr, [](void *) {});
  py::array arr(py::dtype(dtype_name(dt)), std::vector<py::ssize_t>{n},
                std::vector<py::ssize_t>{elem}, s.ptr, base);
  return torch_module().attr("from_numpy")(arr);
}

template <DataType DT>
Span<DT> span_from_tensor(const py::object &t) {
  TensorInfo i = tensor_info(t, "tensor", (int64_t)sizeof_dtype(DT));
  auto keep = std::shared_ptr<void>(new py::object(t), [](void *p) {
    py::gil_scoped_acquire g;
    delete static_cast<py::object *>(p);
  });
  return Span<DT>(i.ptr, i.numel, i.cuda, keep);
}

void span_copy_from(SpanBase &s, int64_t span_bytes, const py::object &t) {
  TensorInfo i = tensor_info(t, "tensor");
  const size_t n = (size_t)std::min<int64_t>(span_bytes, i.numel * i.elem);  // span.h:73-79
  if (n == 0) return;
  if (s.device || i.cuda)
    check_hip("copy into span", gear_hip_memcpy(s.ptr, i.ptr, n));
  else
    std::memcpy(s.ptr, i.ptr, n);
}

template <DataType DT>
void bind_span(py::module_ &m, const char *name) {
  using S = Span<DT>;
  constexpr int64_t kElem = DT == DataType::kFloat16 ? 2 : 0;
  (void)kElem;
  py::class_<S>(m, name)
      .def(py::init([](const py::object &t) { return span_from_tensor<DT>(t); }))
      .def_static("from_tensor", [](const py::object &t) { return span_from_tensor<DT>(t); })
      .def_static("Tensor", [](const S &s) { return span_to_tensor(s, s.size * (int64_t)sizeof_dtype(DT), DT); })
      .def("tensor", [](const S &s) { return span_to_tensor(s, s.size * (int64_t)sizeof_dtype(DT), DT); })
      .def("cast_tensor",
           [](const S &s, DataType dt) { return span_to_tensor(s, s.size * (int64_t)sizeof_dtype(DT), dt); })
      .def("copy", [](S &s, const py::object &t) { span_copy_from(s, s.size * (int64_t)sizeof_dtype(DT), t); })
      .def("copy_to",
           [](const S &s, const py::object &t) {
             TensorInfo i = tensor_info(t, "tensor");
             const size_t n = (size_t)std::min<int64_t>(s.size * (int64_t)sizeof_dtype(DT), i.numel * i.elem);
             if (n) check_hip("copy from span", gear_hip_memcpy(i.ptr, s.ptr, n));
           })
      .def_property_readonly("size", [](const S &s) { return s.size; })
      .def_property_readonly("address", [](const S &s) { return reinterpret_cast<uintptr_t>(s.ptr); })
      .def_property_readonly("is_device", [](const S &s) { return s.device; })
#define AS_(NAME, TDT)                                                                              \
  .def(NAME, [](const S &s) {                                                                        \
    return Span<TDT>(s.ptr, s.size * (int64_t)sizeof_dtype(DT) / (int64_t)sizeof_dtype(TDT), s.device, s.keep); \
  })
      AS_("as_bool", DataType::kBool) AS_("as_int8", DataType::kInt8) AS_("as_uint8", DataType::kUint8)
      AS_("as_int16", DataType::kInt16) AS_("as_int32", DataType::kInt32)
      AS_("as_int64", DataType::kInt64) AS_("as_float32", DataType::kFloat32)
      AS_("as_float64", DataType::kFloat64)
#undef AS_
      ;
  py::implicitly_convertible<py::object, S>();
}

using Int64Span = Span<DataType::kInt64>;
using Uint8Span = Span<DataType::kUint8>;

struct MemoryPtr {
  uintptr_t value;
};

uintptr_t address_of(const py::object &src) {
  if (py::isinstance<MemoryPtr>(src)) return src.cast<MemoryPtr>().value;
  if (py::isinstance<py::int_>(src)) return src.cast<uintptr_t>();
  if (py::hasattr(src, "data_ptr")) return src.attr("data_ptr")().cast<uintptr_t>();
  throw py::type_error("expected a MemoryPtr, an integer address or a tensor");
}

// Python face of a MemoryBlock with a fixed placement (Memory / SharedMemory / CudaMemory / ...)
struct PyMemory {
  std::shared_ptr<MemoryBlock> block;
  PyMemory(size_t size, Placement p, key_t key = 0, bool create = true)
      : block(std::make_shared<MemoryBlock>(size, p, key, create)) {}
};

py::tuple indexset_state_tuple(const IndexsetState &s) {
  py::array_t<uint8_t> bytes((py::ssize_t)s.bytes.size());
  if (!s.bytes.empty()) std::memcpy(bytes.mutable_data(), s.bytes.data(), s.bytes.size());
  return py::make_tuple((int64_t)s.index_offset, (int64_t)s.local_capacity,
                        (int64_t)s.global_capacity, bytes);
}

std::shared_ptr<IndexsetState> indexset_state_from_tuple(const py::tuple &t) {
  if (t.size() != 4) throw std::runtime_error("Invalid state for unpickling IndexsetState");
  const size_t off = (size_t)t[0].cast<int64_t>(), local = (size_t)t[1].cast<int64_t>(),
               global = (size_t)t[2].cast<int64_t>();
  py::array_t<uint8_t, py::array::c_style | py::array::forcecast> mem = t[3].cast<py::array>();
  if ((size_t)mem.size() < local * 12) throw std::runtime_error("IndexsetState blob is too short");
  const uint8_t *p = mem.data();
  return std::make_shared<IndexsetState>(global, local, off, reinterpret_cast<const int64_t *>(p),
                                         reinterpret_cast<const float *>(p + local * 8));
}

Placement placement_from(const std::string &arg) {
  if (!arg.empty() && arg != "auto") return parse_placement(arg);
  const char *env = getenv("GEAR_TABLE_PLACEMENT");
  return parse_placement(env ? env : "auto");
}

struct Handler {
  std::shared_ptr<TrajectoryTable> table;
  StorageHandler impl;
  Handler(std::shared_ptr<TrajectoryTable> t, size_t g, Range w, Range r)
      : table(t), impl(t, g, w, r) {}
};

// the column descriptors of one multi-column gather of `num` windows into dsts (and masks)
std::vector<gear_hip_column_desc> column_descs(Handler &h, int64_t num,
                                               const std::vector<size_t> &columns,
                                               const std::vector<py::object> &dsts, bool zero_fill,
                                               const py::object &masks) {
  if (columns.size() != dsts.size() || columns.size() > GEAR_HIP_MAX_COLUMNS)
    throw std::runtime_error("columns and dsts differ in length (or more than 16 columns)");
  std::vector<gear_hip_column_desc> descs(columns.size());
  for (size_t k = 0; k < columns.size(); ++k) {
    const ColumnWindow w = h.impl.window(columns[k]);
    TensorInfo d = tensor_info(dsts[k], "dst", 0, 1);
    if (d.numel * d.elem < num * w.dst_stride)
      throw std::runtime_error("dst is smaller than the gathered batch");
    descs[k].dst = d.ptr;
    descs[k].mask_out = nullptr;
    if (!masks.is_none()) {
      py::object mk = masks.cast<py::sequence>()[k];
      if (!mk.is_none()) {
        TensorInfo mi = tensor_info(mk, "mask", 1, 1);
        if (mi.numel < num * w.span) throw std::runtime_error("mask is smaller than [num, length]");
        descs[k].mask_out = static_cast<uint8_t *>(mi.ptr);
      }
    }
    descs[k].ofst = w.ofst;
    descs[k].span = w.span;
    descs[k].step_bytes = w.step_bytes;
    descs[k].col_base = w.col_base;
    descs[k].dst_stride = w.dst_stride;
    descs[k].pad_head = w.pad_head ? 1 : 0;
    descs[k].zero_fill = zero_fill ? 1 : 0;
  }
  return descs;
}

}  // namespace

PYBIND11_MODULE(_libgear, libgear) {
  libgear.doc() = "GEAR host library over the MI355X replay-sampling kernels";
  py::module_ m = libgear.def_submodule("core", "Core functional components provided here.");
  py::module_ comm = libgear.def_submodule("comm", "Communicator submodule (not part of this build)");
  comm.def("create_nccl_id", []() -> py::bytes {
    throw std::runtime_error("multi-rank trajectory exchange is not part of this single-GPU build");
  });

  // ---- common: dtypes, ranges, spans (src/common/pybind.cc) ------------------------------------
  py::enum_<DataType>(m, "DataType", py::arithmetic(), "Meta-class for data-type")
      .value("bool", DataType::kBool)
      .value("int8", DataType::kInt8)
      .value("uint8", DataType::kUint8)
      .value("short", DataType::kInt16)
      .value("int16", DataType::kInt16)
      .value("int", DataType::kInt32)
      .value("int32", DataType::kInt32)
      .value("long", DataType::kInt64)
      .value("int64", DataType::kInt64)
      .value("half", DataType::kFloat16)
      .value("float16", DataType::kFloat16)
      .value("float", DataType::kFloat32)
      .value("float32", DataType::kFloat32)
      .value("double", DataType::kFloat64)
      .value("float64", DataType::kFloat64)
      .export_values();
  m.def("sizeof_dtype", &sizeof_dtype);

  py::class_<Range>(m, "Range")
      .def(py::init<size_t, size_t>())
      .def_readwrite("lb", &Range::lb)
      .def_readwrite("hb", &Range::hb);

  bind_span<DataType::kBool>(m, "BoolSpan");
  bind_span<DataType::kInt8>(m, "Int8Span");
  bind_span<DataType::kUint8>(m, "Uint8Span");
  bind_span<DataType::kInt16>(m, "Int16Span");
  bind_span<DataType::kInt32>(m, "Int32Span");
  bind_span<DataType::kInt64>(m, "Int64Span");
  bind_span<DataType::kFloat32>(m, "Float32Span");
  bind_span<DataType::kFloat64>(m, "Float64Span");

  // ---- memory (src/memory/pybind.cc) -----------------------------------------------------------
  py::class_<MemoryPtr>(m, "MemoryPtr")
      .def(py::init([](int64_t a) { return MemoryPtr{(uintptr_t)a}; }))
      .def_property_readonly("address", [](const MemoryPtr &p) { return p.value; })
      .def("__int__", [](const MemoryPtr &p) { return p.value; })
      .def("__repr__", [](const MemoryPtr &p) {
        std::stringstream ss;
        ss << reinterpret_cast<void *>(p.value);
        return ss.str();
      });

  py::class_<PyMemory, std::shared_ptr<PyMemory>> memory_class(m, "Memory");
  py::enum_<Placement>(memory_class, "MemoryType")
      .value("cpu", Placement::kHost)
      .value("uvm", Placement::kPinned)
      .value("shared", Placement::kShm)
      .value("cuda", Placement::kDevice)
      .export_values();
  auto common_memory = [](auto &cls) {
    cls.def("alloc", [](PyMemory &s) { return s.block->alloc(); })
        .def("free", [](PyMemory &s) { return s.block->free(); })
        .def("__repr__", [](const PyMemory &s) { return s.block->to_string(); })
        .def_property_readonly("addr", [](const PyMemory &s) {
          return MemoryPtr{reinterpret_cast<uintptr_t>(s.block->any())};
        })
        .def_property_readonly("size", [](const PyMemory &s) { return s.block->size(); })
        .def_property_readonly("type", [](const PyMemory &s) { return s.block->placement(); });
  };
  memory_class.def(py::init([](size_t size) { return std::make_shared<PyMemory>(size, Placement::kHost); }),
                   py::arg("size"));
  common_memory(memory_class);
  struct PySharedMemory : PyMemory { using PyMemory::PyMemory; };
  struct PyCudaMemory : PyMemory { using PyMemory::PyMemory; };
  struct PyUvMemory : PyMemory { using PyMemory::PyMemory; };
  py::class_<PySharedMemory, std::shared_ptr<PySharedMemory>, PyMemory> shm_class(m, "SharedMemory");
  shm_class.def(py::init([](key_t key, size_t size, bool create) {
                  return std::make_shared<PySharedMemory>(size, Placement::kShm, key, create);
                }),
                py::arg("key"), py::arg("size"), py::arg("create"))
      .def_property_readonly("key", [](const PyMemory &s) { return s.block->key(); })
      .def_property_readonly("create", [](const PyMemory &s) { return s.block->create(); })
      .def_property_readonly("shmid", [](const PyMemory &s) { return s.block->shmid(); });
  py::class_<PyCudaMemory, std::shared_ptr<PyCudaMemory>, PyMemory>(m, "CudaMemory")
      .def(py::init([](size_t size) { return std::make_shared<PyCudaMemory>(size, Placement::kDevice); }),
           py::arg("size"));
  py::class_<PyUvMemory, std::shared_ptr<PyUvMemory>, PyMemory>(m, "CudaUVMemory")
      .def(py::init([](size_t size) { return std::make_shared<PyUvMemory>(size, Placement::kPinned); }),
           py::arg("size"));

  // ---- storage specs (src/storage/pybind.cc:20-70) ----------------------------------------------
  py::class_<ColumnSpec, std::shared_ptr<ColumnSpec>>(m, "ColumnSpec")
      .def(py::init<std::vector<size_t>, DataType, std::string>(), py::arg("shape"),
           py::arg("dtype"), py::arg("name") = "")
      .def_readwrite("dtype", &ColumnSpec::dtype)
      .def_readwrite("shape", &ColumnSpec::shape)
      .def_readwrite("name", &ColumnSpec::name)
      .def("size", &ColumnSpec::size)
      .def(py::pickle([](const ColumnSpec &s) { return py::make_tuple(s.shape, s.dtype, s.name); },
                      [](py::tuple t) {
                        if (t.size() != 3) throw std::runtime_error("Invalid state for ColumnSpec unpickling!");
                        return std::make_shared<ColumnSpec>(t[0].cast<std::vector<size_t>>(),
                                                            t[1].cast<DataType>(),
                                                            t[2].cast<std::string>());
                      }));

  py::class_<TableSpec, std::shared_ptr<TableSpec>>(m, "TableSpec")
      .def(py::init<size_t, size_t, size_t, size_t, size_t, std::vector<ColumnSpec>>())
      .def_readwrite("rank", &TableSpec::rank)
      .def_readwrite("worldsize", &TableSpec::worldsize)
      .def_readwrite("trajectory_length", &TableSpec::trajectory_length)
      .def_readwrite("capacity", &TableSpec::capacity)
      .def_readonly("num_columns", &TableSpec::num_columns)
      .def_readonly("column_specs", &TableSpec::column_specs)
      .def("index", &TableSpec::index)
      .def("size", &TableSpec::size)
      .def(py::pickle(
          [](const TableSpec &s) {
            return py::make_tuple(s.rank, s.worldsize, s.trajectory_length, s.capacity,
                                  s.num_columns, s.column_specs);
          },
          [](py::tuple t) {
            if (t.size() != 6) throw std::runtime_error("Invalid state for TableSpec unpickling!");
            return std::make_shared<TableSpec>(t[0].cast<size_t>(), t[1].cast<size_t>(),
                                               t[2].cast<size_t>(), t[3].cast<size_t>(),
                                               t[4].cast<size_t>(),
                                               t[5].cast<std::vector<ColumnSpec>>());
          }));

  // ---- patterns + handler (src/storage/pybind.cc:72-165) ----------------------------------------
  py::class_<SubscribePattern, std::shared_ptr<SubscribePattern>> pattern(m, "SubscribePattern");
  py::enum_<SubscribePattern::PadOption>(pattern, "PadOption")
      .value("inactive", SubscribePattern::PadOption::kInactive)
      .value("head", SubscribePattern::PadOption::kHead)
      .value("tail", SubscribePattern::PadOption::kTail)
      .export_values();
  pattern.def(py::init<int, size_t, SubscribePattern::PadOption>())
      .def(py::init([](int offset, size_t length) {
        return SubscribePattern(offset, length, SubscribePattern::PadOption::kTail);
      }))
      .def_readonly("offset", &SubscribePattern::offset)
      .def_readonly("length", &SubscribePattern::length)
      .def_readonly("pad_option", &SubscribePattern::pad_option)
      .def("__repr__", &SubscribePattern::to_string)
      .def(py::pickle(
          [](const SubscribePattern &p) { return py::make_tuple(p.offset, p.length, p.pad_option); },
          [](py::tuple t) {
            if (t.size() != 3) throw std::runtime_error("Invalid state for SubscribePattern unpickling");
            return std::make_shared<SubscribePattern>(t[0].cast<int>(), t[1].cast<size_t>(),
                                                      t[2].cast<SubscribePattern::PadOption>());
          }));

  py::class_<TrajectoryTable, std::shared_ptr<TrajectoryTable>>(m, "TrajectoryTable")
      .def(py::init([](const TableSpec &spec, key_t key, bool create, const std::string &placement) {
             return std::make_shared<TrajectoryTable>(spec, key, create, placement_from(placement));
           }),
           py::arg("spec"), py::arg("key"), py::arg("create"), py::arg("placement") = "auto")
      .def_property_readonly("ncolumns", &TrajectoryTable::ncolumns)
      .def("get_table_spec", &TrajectoryTable::table_spec)
      .def("get_column_spec", &TrajectoryTable::column_spec)
      .def("get_address",
           [](TrajectoryTable &t) { return MemoryPtr{reinterpret_cast<uintptr_t>(t.block().any())}; })
      .def("connect", &TrajectoryTable::connect)
      .def_property_readonly("placement", [](TrajectoryTable &t) { return std::string(placement_name(t.block().placement())); })
      .def_property_readonly("device_address", [](TrajectoryTable &t) { return reinterpret_cast<uintptr_t>(t.block().device()); })
      .def_property_readonly("trajectory_stride", &TrajectoryTable::trajectory_stride)
      .def("column_stride", &TrajectoryTable::column_stride)
      .def("column_base", &TrajectoryTable::column_base)
      .def(py::pickle(
          [](const TrajectoryTable &t) {
            const size_t n = t.block().size();
            py::array_t<uint8_t> bytes((py::ssize_t)n);
            if (t.block().any() == nullptr) throw std::runtime_error("cannot pickle a table that is not connected");
            t.block().read(0, bytes.mutable_data(), n);
            return py::make_tuple(t.table_spec(), t.block().key(), n, t.block().create(), bytes);
          },
          [](py::tuple t) {
            if (t.size() != 5) throw std::runtime_error("Invalid state!");
            auto table = std::make_shared<TrajectoryTable>(t[0].cast<TableSpec>(), t[1].cast<key_t>(),
                                                           t[3].cast<bool>(), placement_from("auto"));
            if (table->connect() < 0) throw std::runtime_error("cannot allocate the table memory");
            py::array_t<uint8_t, py::array::c_style | py::array::forcecast> bytes = t[4].cast<py::array>();
            const size_t n = std::min<size_t>(t[2].cast<size_t>(), (size_t)bytes.size());
            table->block().write(0, bytes.data(), std::min(n, table->block().size()));
            return table;
          }));

  auto span64 = [](const py::object &o, const char * /*name*/) {
    if (py::isinstance<Int64Span>(o)) return o.cast<Int64Span>();
    return span_from_tensor<DataType::kInt64>(o);
  };
  auto do_sub = [span64](Handler &h, const py::object &idxs, const py::object &tss,
                         const py::object &lens, size_t column, const py::object &so,
                         const py::object &dof, const py::object &cl) {
    Int64Span a = span64(idxs, "indices"), b = span64(tss, "timesteps"), c = span64(lens, "lengths");
    Int64Span x = span64(so, "src_offsets"), y = span64(dof, "dst_offsets"), z = span64(cl, "lengths");
    if (a.size != b.size || a.size != c.size)
      throw std::runtime_error("Spans describing target propoties has inconsistent size!");
    if (a.size > x.size || a.size > y.size || a.size > z.size)
      throw std::runtime_error("Spans describing target propoties larger than destination spans, potential overrun!");
    if (a.device || b.device || c.device || x.device || y.device || z.device)
      throw std::runtime_error("sub() works on host tensors; use subcopy() for device tensors");
    return h.impl.sub(a.size, static_cast<const int64_t *>(a.ptr), static_cast<const int64_t *>(b.ptr),
                      static_cast<const int64_t *>(c.ptr), column, static_cast<int64_t *>(x.ptr),
                      static_cast<int64_t *>(y.ptr), static_cast<int64_t *>(z.ptr));
  };

  py::class_<Handler, std::shared_ptr<Handler>>(m, "CpuTrajectoryStorageHandler")
      .def("set", [](Handler &h, std::vector<size_t> cids, const std::vector<SubscribePattern> &p) { h.impl.set(cids, p); })
      .def("sub", do_sub)
      .def("sub_", do_sub)
      .def("subcopy",
           [](Handler &h, const py::object &idxs, const py::object &tss, const py::object &lens,
              size_t column, const py::object &dst, bool zero_fill, const py::object &mask) {
             const ColumnWindow w = h.impl.window(column);
             TensorInfo a = tensor_info(idxs, "indices", 8, 1), b = tensor_info(tss, "timesteps", 8, 1),
                        c = tensor_info(lens, "lengths", 8, 1), d = tensor_info(dst, "dst", 0, 1);
             if (a.numel != b.numel || a.numel != c.numel)
               throw std::runtime_error("indices, timesteps and lengths differ in size");
             if (d.numel * d.elem < a.numel * w.dst_stride)
               throw std::runtime_error("dst is smaller than the gathered batch");
             uint8_t *mp = nullptr;
             if (!mask.is_none()) {
               TensorInfo mi = tensor_info(mask, "mask", 1, 1);
               if (mi.numel < a.numel * w.span) throw std::runtime_error("mask is smaller than [num, length]");
               mp = static_cast<uint8_t *>(mi.ptr);
             }
             // one-column form of the checked launch: the handler knows the table's extent, so
             // an index outside it gathers nothing instead of reading outside the table
             gear_hip_column_desc desc;
             desc.dst = d.ptr;
             desc.mask_out = mp;
             desc.ofst = w.ofst;
             desc.span = w.span;
             desc.step_bytes = w.step_bytes;
             desc.col_base = w.col_base;
             desc.dst_stride = w.dst_stride;
             desc.pad_head = w.pad_head ? 1 : 0;
             desc.zero_fill = zero_fill ? 1 : 0;
             check_hip("subcopy",
                       gear_hip_subcopy_multi_checked(
                           h.impl.device_base(), a.numel, static_cast<const int64_t *>(a.ptr),
                           static_cast<const int64_t *>(b.ptr), static_cast<const int64_t *>(c.ptr),
                           (int64_t)h.impl.table().trajectory_stride(),
                           (int64_t)h.impl.table().table_spec().capacity,
                           (int64_t)h.impl.table().table_spec().trajectory_length, &desc, 1,
                           current_stream()));
           },
           py::arg("indices"), py::arg("timesteps"), py::arg("lengths"), py::arg("column"),
           py::arg("dst"), py::arg("zero_fill") = false, py::arg("mask") = py::none())
      .def("subcopy_multi",
           [](Handler &h, const py::object &idxs, const py::object &tss, const py::object &lens,
              const std::vector<size_t> &columns, const std::vector<py::object> &dsts, bool zero_fill,
              const py::object &masks) {
             TensorInfo a = tensor_info(idxs, "indices", 8, 1), b = tensor_info(tss, "timesteps", 8, 1),
                        c = tensor_info(lens, "lengths", 8, 1);
             if (a.numel != b.numel || a.numel != c.numel)
               throw std::runtime_error("indices, timesteps and lengths differ in size");
             const std::vector<gear_hip_column_desc> descs =
                 column_descs(h, a.numel, columns, dsts, zero_fill, masks);
             check_hip("subcopy_multi",
                       gear_hip_subcopy_multi_checked(
                           h.impl.device_base(), a.numel, static_cast<const int64_t *>(a.ptr),
                           static_cast<const int64_t *>(b.ptr), static_cast<const int64_t *>(c.ptr),
                           (int64_t)h.impl.table().trajectory_stride(),
                           (int64_t)h.impl.table().table_spec().capacity,
                           (int64_t)h.impl.table().table_spec().trajectory_length, descs.data(),
                           (int)descs.size(), current_stream()));
           },
           py::arg("indices"), py::arg("timesteps"), py::arg("lengths"), py::arg("columns"),
           py::arg("dsts"), py::arg("zero_fill") = true, py::arg("masks") = py::none())
      // One call for a loader step after the draws (no reference counterpart as a binding: it is
      // OfflineLoader.fused_iterate, gear/loader/offline_loader.py:155-204, from the sort of the
      // sampled indices to the last column's subcopy): the batch is selected and looked up --
      //   kind "weighted"   draws = fp32 uniforms in [0, 1), searched in `prefix` (fp64)
      //   kind "uniform"    draws = int64 positions into `indices`
      //   kind "positions"  draws = int64 positions already in batch order (a top-k selection)
      // sorted (not for "positions"), sampled = indices[position], local = sampled - index_offset,
      // lens = timesteps[local] -- and all columns are gathered with the offline convention
      // timestep == length (offline_loader.py:200-201), everything enqueued on the current stream.
      // `indices` must ascend (then sorting positions sorts the sampled indices).
      .def("select_subcopy",
           [](Handler &h, const std::string &kind, const py::object &draws, const py::object &prefix,
              const py::object &indices, int64_t index_offset, const py::object &timesteps,
              const std::vector<size_t> &columns, const std::vector<py::object> &dsts, bool zero_fill,
              const py::object &masks, const py::object &sampled_out, const py::object &local_out,
              const py::object &lens_out) {
             TensorInfo it = tensor_info(indices, "indices", 8, 1),
                        tt = tensor_info(timesteps, "timesteps", 8, 1),
                        so = tensor_info(sampled_out, "sampled_out", 8, 1),
                        lo = tensor_info(local_out, "local_out", 8, 1),
                        le = tensor_info(lens_out, "lens_out", 8, 1);
             void *st = current_stream();
             int64_t num = 0;
             if (kind == "weighted") {
               TensorInfo d = tensor_info(draws, "draws", 4, 1), p = tensor_info(prefix, "prefix", 8, 1);
               num = d.numel;
               if (p.numel != it.numel) throw std::runtime_error("prefix and indices differ in length");
               if (so.numel < num || lo.numel < num || le.numel < num)
                 throw std::runtime_error("an output is smaller than the batch");
               size_t have = 0;
               void *ws = workspace("sample", st, gear_hip_sample_workspace_bytes(num), &have);
               check_hip("select_subcopy (sample)",
                         gear_hip_sample_lookup_f64(
                             static_cast<const double *>(p.ptr), p.numel, static_cast<const float *>(d.ptr),
                             num, 1, static_cast<const int64_t *>(it.ptr), index_offset,
                             static_cast<const int64_t *>(tt.ptr), tt.numel, static_cast<int64_t *>(so.ptr),
                             static_cast<int64_t *>(lo.ptr), static_cast<int64_t *>(le.ptr), ws, have, st));
             } else if (kind == "uniform" || kind == "positions") {
               TensorInfo d = tensor_info(draws, "draws", 8, 1);
               num = d.numel;
               if (so.numel < num || lo.numel < num || le.numel < num)
                 throw std::runtime_error("an output is smaller than the batch");
               if (kind == "uniform") {
                 size_t have = 0;
                 void *ws = workspace("sample", st, gear_hip_sample_workspace_bytes(num), &have);
                 check_hip("select_subcopy (sort)",
                           gear_hip_sort_lookup_i64(
                               static_cast<const int64_t *>(d.ptr), num, it.numel > 0 ? it.numel : 1,
                               static_cast<const int64_t *>(it.ptr), it.numel, index_offset,
                               static_cast<const int64_t *>(tt.ptr), tt.numel, static_cast<int64_t *>(so.ptr),
                               static_cast<int64_t *>(lo.ptr), static_cast<int64_t *>(le.ptr), ws, have, st));
               } else {
                 check_hip("select_subcopy (look-up)",
                           gear_hip_lookup_i64(static_cast<const int64_t *>(d.ptr), num,
                                               static_cast<const int64_t *>(it.ptr), it.numel, index_offset,
                                               static_cast<const int64_t *>(tt.ptr), tt.numel,
                                               static_cast<int64_t *>(so.ptr), static_cast<int64_t *>(lo.ptr),
                                               static_cast<int64_t *>(le.ptr), st));
               }
             } else {
               throw std::invalid_argument("kind must be 'weighted', 'uniform' or 'positions'");
             }
             if (num == 0) return;
             const std::vector<gear_hip_column_desc> descs =
                 column_descs(h, num, columns, dsts, zero_fill, masks);
             check_hip("select_subcopy (gather)",
                       gear_hip_subcopy_multi_checked(
                           h.impl.device_base(), num, static_cast<const int64_t *>(lo.ptr),
                           static_cast<const int64_t *>(le.ptr), static_cast<const int64_t *>(le.ptr),
                           (int64_t)h.impl.table().trajectory_stride(),
                           (int64_t)h.impl.table().table_spec().capacity,
                           (int64_t)h.impl.table().table_spec().trajectory_length, descs.data(),
                           (int)descs.size(), st));
           },
           py::arg("kind"), py::arg("draws"), py::arg("prefix"), py::arg("indices"),
           py::arg("index_offset"), py::arg("timesteps"), py::arg("columns"), py::arg("dsts"),
           py::arg("zero_fill"), py::arg("masks"), py::arg("sampled_out"), py::arg("local_out"),
           py::arg("lens_out"))
      .def("view",
           [](Handler &h, size_t index, size_t column) {
             size_t off, len;
             h.impl.view_range(index, column, &off, &len);
             MemoryBlock &b = h.table->block();
             if (b.any() == nullptr) throw std::runtime_error("table memory is not connected");
             if (off + len > b.size()) throw std::out_of_range("trajectory index outside the table");
             return Uint8Span(static_cast<char *>(b.any()) + off, (int64_t)len, b.host() == nullptr, h.table);
           })
      .def("raw",
           [](Handler &h, size_t offset, size_t length) {
             MemoryBlock &b = h.table->block();
             if (b.any() == nullptr) throw std::runtime_error("table memory is not connected");
             if (offset + length > b.size()) throw std::out_of_range("range outside the table");
             return Uint8Span(static_cast<char *>(b.any()) + offset, (int64_t)length, b.host() == nullptr, h.table);
           })
      .def("connect", [](Handler &, int, int, py::bytes) {
        throw std::runtime_error("NCCL trajectory exchange is not part of this single-GPU build");
      })
      .def("subsend", [](Handler &, py::args) {
        throw std::runtime_error("NCCL trajectory exchange is not part of this single-GPU build");
      })
      .def("subrecv", [](Handler &, py::args) {
        throw std::runtime_error("NCCL trajectory exchange is not part of this single-GPU build");
      });

  m.def("get_cpu_handler",
        [](std::shared_ptr<TrajectoryTable> table, size_t global_capacity, Range w, Range r) {
          return std::make_shared<Handler>(table, global_capacity, w, r);
        });

  // ---- index set (src/index/pybind.cc:293-356) ---------------------------------------------------
  py::class_<IndexsetState, std::shared_ptr<IndexsetState>>(m, "IndexsetState")
      .def_readonly("global_capacity", &IndexsetState::global_capacity)
      .def_readonly("local_capacity", &IndexsetState::local_capacity)
      .def_readonly("index_offset", &IndexsetState::index_offset)
      .def(py::pickle([](const IndexsetState &s) { return indexset_state_tuple(s); },
                      [](py::tuple t) { return indexset_state_from_tuple(t); }));

  py::class_<Indexset, std::shared_ptr<Indexset>>(m, "Indexset")
      .def(py::init([](double g, double l, double off, bool shared, key_t key, bool create) {
             // the reference's dataset passes float capacities (capacity / shard_world)
             return std::make_shared<Indexset>((size_t)g, (size_t)l, (size_t)off, shared, key, create);
           }),
           py::arg("global_capacity"), py::arg("local_capacity"), py::arg("index_offet"),
           py::arg("shared") = false, py::arg("key") = 0, py::arg("create") = false)
      .def(py::init([](double g, double l, double index_offset, bool shared, key_t key, bool create) {
             return std::make_shared<Indexset>((size_t)g, (size_t)l, (size_t)index_offset, shared, key, create);
           }),
           py::arg("global_capacity"), py::arg("local_capacity"), py::kw_only(),
           py::arg("index_offset"), py::arg("shared") = false, py::arg("key") = 0,
           py::arg("create") = false)
      .def_static("load_state",
                  [](IndexsetState &s, bool shared, key_t key, bool create) {
                    return std::make_shared<Indexset>(s, shared, key, create);
                  })
      .def_property_readonly("timesteps",
                             [](std::shared_ptr<Indexset> self) {
                               SpanBase s;
                               s.ptr = self->timesteps();
                               s.keep = self;
                               return span_to_tensor(s, (int64_t)self->local_capacity() * 8, DataType::kInt64);
                             })
      .def_property_readonly("weights",
                             [](std::shared_ptr<Indexset> self) {
                               SpanBase s;
                               s.ptr = self->weights();
                               s.keep = self;
                               return span_to_tensor(s, (int64_t)self->local_capacity() * 4, DataType::kFloat32);
                             })
      .def("set_timestep", &Indexset::set_timestep)
      .def("set_weight", &Indexset::set_weight)
      .def_property_readonly("global_capacity", &Indexset::global_capacity)
      .def_property_readonly("local_capacity", &Indexset::local_capacity)
      .def_property_readonly("capacity", &Indexset::local_capacity)
      .def_property_readonly("index_offset", &Indexset::index_offset)
      .def_property_readonly("is_sharing", &Indexset::is_sharing)
      .def_property_readonly("shm_key", &Indexset::shm_key)
      .def_property_readonly("device_weights_address",
                             [](const Indexset &s) { return reinterpret_cast<uintptr_t>(s.device_weights()); })
      .def("get_state", [](Indexset &s) { return std::make_shared<IndexsetState>(s.get_state()); });

  // ---- request arrays of the online path (src/index/pybind.cc:154-206) -------------------------
  py::class_<InferenceRequestArray>(m, "InferenceRequestArray")
      .def_readonly("count", &InferenceRequestArray::count)
      .def("insert", &InferenceRequestArray::insert)
      .def("clear", &InferenceRequestArray::clear)
      .def("source_element_view", [](InferenceRequestArray &a, size_t i) { return a.srcs[i]; })
      .def("index_element_view", [](InferenceRequestArray &a, size_t i) { return a.idxs[i]; })
      .def("timestep_element_view", [](InferenceRequestArray &a, size_t i) { return a.tss[i]; })
      .def("source_tensor_view",
           [](InferenceRequestArray &a) {
             SpanBase s;
             s.ptr = a.srcs;
             return span_to_tensor(s, (int64_t)a.count * 4, DataType::kInt32);
           }, py::keep_alive<0, 1>())
      .def("index_tensor_view",
           [](InferenceRequestArray &a) {
             SpanBase s;
             s.ptr = a.idxs;
             return span_to_tensor(s, (int64_t)a.count * 8, DataType::kInt64);
           }, py::keep_alive<0, 1>())
      .def("timestep_tensor_view",
           [](InferenceRequestArray &a) {
             SpanBase s;
             s.ptr = a.tss;
             return span_to_tensor(s, (int64_t)a.count * 8, DataType::kInt64);
           }, py::keep_alive<0, 1>());

  py::class_<WeightUpdateRequestArray>(m, "WeightUpdateRequestArray")
      .def_readonly("count", &WeightUpdateRequestArray::count)
      .def("update", &WeightUpdateRequestArray::update)
      .def("updated_element_view", [](WeightUpdateRequestArray &a, size_t i) { return a.updated.at(i) != 0; })
      .def("timestep_element_view", [](WeightUpdateRequestArray &a, size_t i) { return a.timesteps[i]; })
      .def("weight_element_view", [](WeightUpdateRequestArray &a, size_t i) { return a.weights[i]; });

  py::class_<CachedRequest, std::shared_ptr<CachedRequest>>(m, "CachedRequest")
      .def(py::init<int64_t>())
      .def_readonly("capacity", &CachedRequest::capacity)
      .def_readonly("iarr", &CachedRequest::iarr)
      .def_readonly("warr", &CachedRequest::warr)
      .def("continuous", [](CachedRequest &self, const py::object &idxs, const py::object &weights) {
        TensorInfo a = tensor_info(idxs, "idxs", 8, 0), b = tensor_info(weights, "weights", 4, 0);
        return self.warr.continuous(static_cast<int64_t *>(a.ptr), a.numel,
                                    static_cast<float *>(b.ptr), b.numel);
      });

  // ---- kernel launchers (src/cuda/*.cu tails) ----------------------------------------------------
  m.def("init", [](int device_id) { check_hip("init", gear_hip_set_device(device_id)); });
  m.def("print_environ", []() {
    int n = 0;
    check_hip("device count", gear_hip_device_count(&n));
    printf("%s: %d\n", "visible_device_count", n);
  });
  m.def("print_compile_options", []() { printf("gear_verbose_debug: disable\nbackend: hip gfx950\n"); });

  m.def("copy", [](const py::object &src, const py::object &dst, const py::object &so,
                   const py::object &dof, int64_t stride) {
    TensorInfo d = tensor_info(dst, "dst", 0, 1), a = tensor_info(so, "src_offsets", 8, 1),
               b = tensor_info(dof, "dst_offsets", 8, 1);
    check_hip("copy", gear_hip_copy(reinterpret_cast<void *>(address_of(src)), d.ptr,
                                    std::min(a.numel, b.numel), static_cast<const int64_t *>(a.ptr),
                                    static_cast<const int64_t *>(b.ptr), stride, current_stream()));
  });
  auto vcopy = [](const py::object &src, const py::object &dst, const py::object &so,
                  const py::object &dof, const py::object &strides, int64_t max_stride) {
    TensorInfo d = tensor_info(dst, "dst", 0, 1), a = tensor_info(so, "src_offsets", 8, 1),
               b = tensor_info(dof, "dst_offsets", 8, 1), c = tensor_info(strides, "strides", 8, 1);
    check_hip("vcopy", gear_hip_vcopy(reinterpret_cast<void *>(address_of(src)), d.ptr,
                                      std::min(std::min(a.numel, b.numel), c.numel),
                                      static_cast<const int64_t *>(a.ptr),
                                      static_cast<const int64_t *>(b.ptr),
                                      static_cast<const int64_t *>(c.ptr), max_stride, current_stream()));
  };
  m.def("vcopy", vcopy);
  m.def("copy_debug", vcopy);

  m.def("sum",
        [](const py::object &val, const py::object &out, int) {
          TensorInfo v = tensor_info(val, "val", 4, 1), o = tensor_info(out, "out", 4, 1);
          size_t have = 0;
          void *st = current_stream();
          void *ws = workspace("sum", st, gear_hip_sum_workspace_bytes(v.numel), &have);
          check_hip("sum", gear_hip_sum_f32(static_cast<const float *>(v.ptr), v.numel,
                                            static_cast<float *>(o.ptr), nullptr, ws, have, st));
        },
        py::arg("val"), py::arg("out"), py::arg("stride") = 1);
  m.def("prefix_sum", [](const py::object &input, const py::object &output) {
    TensorInfo in = tensor_info(input, "input", 4, 1), out = tensor_info(output, "output", 0, 1);
    if (out.numel < in.numel) throw std::runtime_error("output is shorter than input");
    size_t have = 0;
    void *st = current_stream();
    void *ws = workspace("scan", st, gear_hip_scan_workspace_bytes(in.numel), &have);
    if (out.elem == 8)
      check_hip("prefix_sum", gear_hip_scan_f32_f64(static_cast<const float *>(in.ptr),
                                                    static_cast<double *>(out.ptr), in.numel, ws, have,
                                                    st));
    else if (out.elem == 4)
      check_hip("prefix_sum", gear_hip_scan_f32_f32(static_cast<const float *>(in.ptr),
                                                    static_cast<float *>(out.ptr), in.numel, ws, have,
                                                    st));
    else
      throw std::runtime_error("output must be a float32 or float64 tensor");
  });
}
