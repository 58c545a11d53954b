// A compiled `c_lib`: the six entry points that python/collcache/torch/adapter.cc:274-281 of the reference registers
// (coll_torch_init, coll_torch_init_t, coll_torch_test, coll_torch_record, coll_torch_lookup_key_t_val_ret,
// coll_torch_create_emb_shm), as a pybind11 extension module over the extern "C" boundary of libcoll_cache.so.
//
// torch is reached through its Python objects: a tensor arrives as a py::object and is asked for data_ptr(), size()
// and dtype, library memory is a torch int8 tensor kept alive until released (the reference's TorchMemHandle,
// adapter.h:37-46), outputs are views of one reused buffer (adapter.cc:205-237).  So the module needs pybind11 and
// the C header only, no ATen and no HIP header, and is built by g++ (python -m ugache_amd.build).
//
// The module keeps a state of its own (dimensions, buffers): a process uses either this module or the Python module
// c_lib.py for these six calls, not both for one cache.  The GIL is released around every call into the library and
// taken again inside the allocator callbacks, which the library may invoke from its own threads.
#include <pybind11/pybind11.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <unordered_map>
#include <vector>

#include "coll_cache_c_api.h"

namespace py = pybind11;

namespace {

constexpr int kF32 = 0, kF16 = 2;  // DataType of coll_cache_lib/common.h (kF32 = 0, kF64 = 1, kF16 = 2) as the C boundary takes it

struct State {
  std::unordered_map<int, int> dev_of_replica;
  size_t external_dim = 0, internal_dim = 0;
  bool two_byte = false;
  py::object external_dtype;  // torch.float32 / torch.float16 / torch.bfloat16
  std::unordered_map<uintptr_t, py::object> held;  // device pointer -> tensor the library holds
  py::object out_buffer;                            // int8 tensor all lookup outputs are views of
  size_t out_capacity_keys = 0;
  std::vector<py::object> host_tables;
  std::vector<void *> host_ptrs;  // tables made by coll_torch_create_emb_shm
};
State *g = nullptr;  // leaked at exit on purpose: its tensors must not be destroyed after the interpreter

py::module_ Torch() { return py::module_::import("torch"); }

std::string Device(int dev_id) { return "cuda:" + std::to_string(dev_id); }

void *Alloc(size_t nbytes, void *user) {
  py::gil_scoped_acquire gil;
  const int dev_id = (int)(intptr_t)user;
  py::object t = Torch().attr("empty")(py::make_tuple(nbytes ? nbytes : 1), py::arg("dtype") = Torch().attr("int8"),
                                       py::arg("device") = Device(dev_id));
  const uintptr_t p = t.attr("data_ptr")().cast<uintptr_t>();
  g->held[p] = t;
  return reinterpret_cast<void *>(p);
}

void Release(void *ptr, void *) {
  py::gil_scoped_acquire gil;
  g->held.erase(reinterpret_cast<uintptr_t>(ptr));
}

void *CurrentStream(int dev_id) {
  py::object s = Torch().attr("cuda").attr("current_stream")(dev_id);
  return reinterpret_cast<void *>(s.attr("cuda_stream").cast<uintptr_t>());
}

void SetupDims(size_t dim, bool two_byte, py::object dtype) {
  g->external_dim = dim;
  g->two_byte = two_byte;
  if (two_byte) {
    if (dim % 2 != 0) {
      fprintf(stderr, "dimension must be even\n");
      abort();
    }
    g->external_dtype = dtype.is_none() ? Torch().attr("float16") : dtype;
    g->internal_dim = dim / 2;
  } else {
    g->external_dtype = Torch().attr("float32");
    g->internal_dim = dim;
  }
}

void Init(int replica_id, size_t key_space_size, int dev_id, uintptr_t cpu_data, size_t dim, double cache_percentage,
          bool two_byte, py::object dtype) {
  Torch().attr("cuda").attr("set_device")(dev_id);
  g->dev_of_replica[replica_id] = dev_id;
  SetupDims(dim, two_byte, dtype);
  void *stream = CurrentStream(dev_id);
  py::gil_scoped_release nogil;
  coll_cache_init_c(replica_id, key_space_size, Alloc, Release, (void *)(intptr_t)dev_id,
                    reinterpret_cast<void *>(cpu_data), two_byte ? kF16 : kF32, dim, cache_percentage, stream);
}

// adapter.cc:126-149
void coll_torch_init(int replica_id, size_t key_space_size, int dev_id, uintptr_t cpu_data, size_t dim,
                     double cache_percentage, bool use_fp16) {
  Init(replica_id, key_space_size, dev_id, cpu_data, dim, cache_percentage, use_fp16, py::none());
}

// adapter.cc:151-190
void coll_torch_init_t(int replica_id, int dev_id, py::object emb, double cache_percentage) {
  py::object dtype = emb.attr("dtype");
  const bool two_byte = dtype.equal(Torch().attr("float16")) || dtype.equal(Torch().attr("bfloat16"));
  if (!two_byte && !dtype.equal(Torch().attr("float32")))
    throw py::type_error("embedding table must be float32, float16 or bfloat16");
  const size_t rows = emb.attr("size")(0).cast<size_t>(), dim = emb.attr("size")(1).cast<size_t>();
  g->host_tables.push_back(emb);  // the library reads the table in place for as long as the cache lives
  Init(replica_id, rows, dev_id, emb.attr("data_ptr")().cast<uintptr_t>(), dim, cache_percentage, two_byte,
       two_byte ? dtype : py::none());
}

int DeviceOf(int replica_id) {
  auto it = g->dev_of_replica.find(replica_id);
  return it == g->dev_of_replica.end() ? 0 : it->second;
}

// adapter.cc:192-203: an uninitialised tensor of the output's shape
py::object coll_torch_test(int replica_id, py::object key) {
  return Torch().attr("empty")(py::make_tuple(key.attr("size")(0), g->external_dim),
                               py::arg("dtype") = Torch().attr("float32"),
                               py::arg("device") = Device(DeviceOf(replica_id)));
}

// adapter.cc:205-237: the rows of `key` in a view of the reused output buffer, [ceil8(n) or n, dim]
py::object coll_torch_lookup_key_t_val_ret(int replica_id, py::object key, bool pad_to_8) {
  const int dev_id = DeviceOf(replica_id);
  py::object kd = key.attr("dtype");
  const bool wide = kd.equal(Torch().attr("int64"));
  if (!wide && !kd.equal(Torch().attr("int32")) && !(py::hasattr(Torch(), "uint32") && kd.equal(Torch().attr("uint32"))))
    throw py::type_error("keys must be int32 / uint32 or int64");
  if (!key.attr("is_cuda").cast<bool>())
    throw py::value_error("keys must live on the GPU (the reference reads key.data_ptr() from device code too)");
  if (!key.attr("is_contiguous")().cast<bool>()) key = key.attr("contiguous")();
  const size_t n = key.attr("size")(0).cast<size_t>();
  const size_t padded = pad_to_8 ? (n + 7) / 8 * 8 : n;
  const size_t row_bytes = g->internal_dim * 4;
  if (padded > g->out_capacity_keys || g->out_buffer.is_none() || !g->out_buffer) {
    size_t max_keys = coll_cache_max_num_keys();
    if (padded > max_keys) {
      fprintf(stderr, "Warning, found a larger batch, re allocating emb output now %zu %zu\n", padded, max_keys);
      max_keys = padded;
    }
    max_keys = (size_t)(max_keys * 1.05) + 8;
    coll_cache_set_max_num_keys(max_keys);
    g->out_buffer = Torch().attr("empty")(py::make_tuple(max_keys * row_bytes), py::arg("dtype") = Torch().attr("int8"),
                                          py::arg("device") = Device(dev_id));
    g->out_capacity_keys = max_keys;
  }
  py::object out = g->out_buffer.attr("__getitem__")(py::slice(0, (py::ssize_t)(padded * row_bytes), 1))
                       .attr("view")(g->external_dtype)
                       .attr("view")(padded, g->external_dim);
  const uintptr_t key_ptr = key.attr("data_ptr")().cast<uintptr_t>();
  const uintptr_t out_ptr = out.attr("data_ptr")().cast<uintptr_t>();
  void *stream = CurrentStream(dev_id);
  {
    py::gil_scoped_release nogil;
    if (wide)
      coll_cache_lookup_i64(replica_id, reinterpret_cast<const int64_t *>(key_ptr), n, reinterpret_cast<void *>(out_ptr),
                            stream);
    else
      coll_cache_lookup(replica_id, reinterpret_cast<uint32_t *>(key_ptr), n, reinterpret_cast<void *>(out_ptr),
                        stream);
  }
  return out;
}

// adapter.cc:270-272: hotness of a batch of keys (a CPU tensor)
void coll_torch_record(int replica_id, py::object key) {
  if (key.attr("is_cuda").cast<bool>()) throw py::value_error("coll_torch_record takes a CPU tensor");
  if (!key.attr("is_contiguous")().cast<bool>()) key = key.attr("contiguous")();
  const bool wide = key.attr("dtype").equal(Torch().attr("int64"));
  const uintptr_t p = key.attr("data_ptr")().cast<uintptr_t>();
  const size_t n = key.attr("numel")().cast<size_t>();
  py::gil_scoped_release nogil;
  if (wide) coll_cache_record_i64(replica_id, reinterpret_cast<const int64_t *>(p), n);
  else coll_cache_record(replica_id, reinterpret_cast<uint32_t *>(p), n);
}

// adapter.cc:239-268: the host table as a CPU tensor [num_key, dim]; pinned and GPU-mapped here (the reference puts
// it into POSIX shared memory and page-locks it later), read from `fname` when one is given
py::object coll_torch_create_emb_shm(int replica_id, size_t num_key, size_t dim, py::object dtype, std::string fname) {
  (void)replica_id;
  const size_t elem = Torch().attr("empty")(py::make_tuple(0), py::arg("dtype") = dtype).attr("element_size")().cast<size_t>();
  const size_t nbytes = num_key * dim * elem;
  void *p = coll_cache_alloc_host_table(nbytes > 64 ? nbytes : 64);
  g->host_ptrs.push_back(p);
  py::module_ ctypes = py::module_::import("ctypes");
  py::object buf = (ctypes.attr("c_uint8").attr("__mul__")(nbytes > 64 ? nbytes : 64)).attr("from_address")(reinterpret_cast<uintptr_t>(p));
  py::object tensor = Torch().attr("frombuffer")(buf, py::arg("dtype") = dtype, py::arg("count") = num_key * dim)
                          .attr("view")(num_key, dim);
  if (!fname.empty()) {
    FILE *f = fopen(fname.c_str(), "rb");
    long size = -1;
    if (f && fseek(f, 0, SEEK_END) == 0) size = ftell(f);
    if (!f || size < 0 || (size_t)size != nbytes) {
      fprintf(stderr, "feat file on disk not equal with claimed shape %ld != %zux%zux%zu\n", size, elem, num_key, dim);
      abort();
    }
    rewind(f);
    const size_t got = fread(p, 1, nbytes, f);
    fclose(f);
    if (got != nbytes) {
      fprintf(stderr, "short read of %s\n", fname.c_str());
      abort();
    }
  }
  return tensor;
}

// not in the reference: drops the cache and every buffer this module holds (tests build several caches per process)
void coll_torch_shutdown() {
  Torch().attr("cuda").attr("synchronize")();
  {
    py::gil_scoped_release nogil;
    coll_cache_shutdown();
  }
  g->held.clear();
  g->out_buffer = py::none();
  g->out_capacity_keys = 0;
  g->host_tables.clear();
  g->dev_of_replica.clear();
  for (void *p : g->host_ptrs) coll_cache_free_host_table(p);  // the tensors over them must not be used from here on
  g->host_ptrs.clear();
}

}  // namespace

PYBIND11_MODULE(c_lib_native, m) {
  g = new State;
  g->out_buffer = py::none();
  m.doc() = "compiled form of collcache.torch.c_lib: the reference's six coll_torch_* entry points over libcoll_cache.so";
  m.def("coll_torch_init", &coll_torch_init);
  m.def("coll_torch_init_t", &coll_torch_init_t);
  m.def("coll_torch_test", &coll_torch_test);
  m.def("coll_torch_record", &coll_torch_record);
  m.def("coll_torch_lookup_key_t_val_ret", &coll_torch_lookup_key_t_val_ret);
  m.def("coll_torch_create_emb_shm", &coll_torch_create_emb_shm, py::arg("replica_id"), py::arg("num_key"),
        py::arg("dim"), py::arg("dtype"), py::arg("fname") = std::string());
  m.def("coll_torch_shutdown", &coll_torch_shutdown);
}
