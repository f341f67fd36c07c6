// Host side of the usual call of HipLoRABackend.add_lora (nanovllm_voxcpm_amd/lora.py), in C++.
//
// The backend mirrors the reference's LoRABackend.add_lora (reference: nanovllm_voxcpm/lora.py:43-54,
// body :241-381): one Python call per LoRA linear and step.  Such a call costs the interpreter
// several microseconds of tensor attribute reads and checks before the launch, which takes about
// four; a decode step of 96 calls is then bound by the host, not by the GPU.  This module does the
// same reads and checks on the tensors' C++ objects.  It decides nothing by itself: it handles a
// call only when everything the Python path would look up for it is what the Python path looked up
// last time (the argument block of these weight buffers, the plan of this step's slot vector, the
// scratch buffer of this stream), fills the per-step fields of the block and calls mlora_add_lora.
// Everything else - a first call, another step, a capture in progress, anything that has to raise
// - is answered with "not handled", and the Python path runs as if this module did not exist, then
// tells it what it found (register_site, set_step, set_scratch).
//
// One state object per backend and thread; every function runs under the interpreter lock.
#include <Python.h>

#include <ATen/core/Tensor.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/csrc/autograd/python_variable.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "mlora.h"

namespace {

constexpr long kNotHandled = 1;  // what call() returns when the Python path has to run

struct Site {
  MloraAddArgs* args = nullptr;
  PyObject* keep = nullptr;  // the object that owns the block
  int k = 0, rank = 0, num_slots = 0, num_slices = 0, device = 0, form = 0, dtype_code = 0;
  bool vectorisable = false;
  c10::ScalarType dtype = c10::ScalarType::Undefined;
  std::vector<int64_t> widths;
};

struct State {
  int (*add_lora)(const MloraAddArgs*) = nullptr;
  size_t (*workspace_bytes)(int32_t, int32_t, int32_t, int32_t) = nullptr;
  std::unordered_map<std::string, Site> sites;
  // what the last call of the Python path looked up for its step
  const PyObject* metadata = nullptr;
  const PyObject* source = nullptr;
  uint32_t version = 0;
  void* stream = nullptr;
  int num_slots = 0;
  int64_t rows = -1;
  const void* plan = nullptr;
  // the eager scratch buffer of a stream
  void* sc_stream = nullptr;
  int sc_device = -1;
  void* sc_ptr = nullptr;
  int64_t sc_bytes = 0;
  // bytes of scratch a shape asks for
  std::unordered_map<uint64_t, int64_t> need;
  long long handled = 0, passed_on = 0;  // calls enqueued here / left to the Python path

  ~State() {
    for (auto& kv : sites) Py_XDECREF(kv.second.keep);
  }
};

const char* kCapsule = "mlora.fastcall.state";

State* state_of(PyObject* capsule) { return static_cast<State*>(PyCapsule_GetPointer(capsule, kCapsule)); }

void destroy(PyObject* capsule) { delete static_cast<State*>(PyCapsule_GetPointer(capsule, kCapsule)); }

// Key of a set of weight buffers: address and shape of every A and B slice, and the element type.
// False when something in the lists is not a contiguous tensor.
bool weights_key(PyObject* a_list, PyObject* b_list, Py_ssize_t n, std::string* key, const at::Tensor** a0) {
  int64_t buf[2 * MLORA_MAX_SLICES * 5 + 1];
  int at = 0;
  for (PyObject* list : {a_list, b_list}) {
    for (Py_ssize_t i = 0; i < n; ++i) {
      PyObject* o = PySequence_Fast_GET_ITEM(list, i);
      if (!THPVariable_Check(o)) return false;
      const at::Tensor& t = THPVariable_Unpack(o);
      if (t.dim() != 3 || !t.is_contiguous()) return false;
      if (list == a_list && i == 0) *a0 = &t;
      buf[at++] = reinterpret_cast<int64_t>(t.data_ptr());
      buf[at++] = t.size(0);
      buf[at++] = t.size(1);
      buf[at++] = t.size(2);
    }
  }
  buf[at++] = static_cast<int64_t>((*a0)->scalar_type());
  key->assign(reinterpret_cast<const char*>(buf), static_cast<size_t>(at) * sizeof(int64_t));
  return true;
}

struct Ref {  // an owned reference, given back at the end of the scope
  PyObject* p;
  ~Ref() { Py_XDECREF(p); }
};

bool on_device(const at::Tensor& t, int device) { return t.is_cuda() && t.device().index() == device; }

PyObject* py_create(PyObject*, PyObject* args) {
  unsigned long long add = 0, ws = 0;
  if (!PyArg_ParseTuple(args, "KK", &add, &ws)) return nullptr;
  State* s = new State();
  s->add_lora = reinterpret_cast<int (*)(const MloraAddArgs*)>(static_cast<uintptr_t>(add));
  s->workspace_bytes = reinterpret_cast<size_t (*)(int32_t, int32_t, int32_t, int32_t)>(static_cast<uintptr_t>(ws));
  return PyCapsule_New(s, kCapsule, destroy);
}

// register_site(state, a_list, b_list, widths, block address, block owner, vectorisable)
PyObject* py_register_site(PyObject*, PyObject* args) {
  PyObject *cap, *a_list, *b_list, *widths, *keep;
  unsigned long long addr = 0;
  int vectorisable = 0;
  if (!PyArg_ParseTuple(args, "OOOOKOp", &cap, &a_list, &b_list, &widths, &addr, &keep, &vectorisable)) return nullptr;
  State* s = state_of(cap);
  if (!s) return nullptr;
  PyObject* af = PySequence_Fast(a_list, "lora_a slices");
  PyObject* bf = af ? PySequence_Fast(b_list, "lora_b slices") : nullptr;
  PyObject* wf = bf ? PySequence_Fast(widths, "widths") : nullptr;
  bool ok = false;
  if (wf) {
    const Py_ssize_t n = PySequence_Fast_GET_SIZE(af);
    std::string key;
    const at::Tensor* a0 = nullptr;
    if (n >= 1 && n <= MLORA_MAX_SLICES && PySequence_Fast_GET_SIZE(bf) == n && PySequence_Fast_GET_SIZE(wf) == n &&
        weights_key(af, bf, n, &key, &a0) && a0->is_cuda()) {
      Site site;
      site.args = reinterpret_cast<MloraAddArgs*>(static_cast<uintptr_t>(addr));
      site.k = site.args->k; site.rank = site.args->r; site.num_slots = site.args->num_slots; site.num_slices = site.args->num_slices;
      site.form = site.args->form; site.dtype_code = site.args->dtype;
      site.device = a0->device().index();
      site.dtype = a0->scalar_type();
      site.vectorisable = vectorisable != 0;
      ok = site.num_slices == n;
      for (Py_ssize_t i = 0; ok && i < n; ++i) {
        const long long w = PyLong_AsLongLong(PySequence_Fast_GET_ITEM(wf, i));
        if (w == -1 && PyErr_Occurred()) { PyErr_Clear(); ok = false; }
        site.widths.push_back(w);
      }
      if (ok) {
        auto it = s->sites.find(key);
        if (it != s->sites.end()) {
          Py_XDECREF(it->second.keep);
          s->sites.erase(it);
        }
        Py_INCREF(keep);
        site.keep = keep;
        s->sites.emplace(std::move(key), std::move(site));
      }
    }
  }
  Py_XDECREF(wf); Py_XDECREF(bf); Py_XDECREF(af);
  if (PyErr_Occurred()) return nullptr;
  return PyBool_FromLong(ok);
}

PyObject* py_clear_sites(PyObject*, PyObject* cap) {
  State* s = state_of(cap);
  if (!s) return nullptr;
  for (auto& kv : s->sites) Py_XDECREF(kv.second.keep);
  s->sites.clear();
  Py_RETURN_NONE;
}

// set_step(state, metadata, source, version, stream, num_slots, rows, plan address): what a call
// outside any capture looked up; the caller keeps metadata, source and the plan alive for as long
// as this stands.  forget_step(state) withdraws it.
PyObject* py_set_step(PyObject*, PyObject* args) {
  PyObject *cap, *metadata, *source;
  unsigned long version = 0;
  unsigned long long stream = 0, plan = 0;
  int num_slots = 0;
  long long rows = 0;
  if (!PyArg_ParseTuple(args, "OOOkKiLK", &cap, &metadata, &source, &version, &stream, &num_slots, &rows, &plan)) return nullptr;
  State* s = state_of(cap);
  if (!s) return nullptr;
  s->metadata = metadata; s->source = source; s->version = static_cast<uint32_t>(version);
  s->stream = reinterpret_cast<void*>(static_cast<uintptr_t>(stream));
  s->num_slots = num_slots; s->rows = rows;
  s->plan = reinterpret_cast<const void*>(static_cast<uintptr_t>(plan));
  Py_RETURN_NONE;
}

PyObject* py_forget_step(PyObject*, PyObject* cap) {
  State* s = state_of(cap);
  if (!s) return nullptr;
  s->metadata = nullptr; s->source = nullptr; s->rows = -1; s->plan = nullptr;
  Py_RETURN_NONE;
}

// set_scratch(state, device index, stream, address, bytes): the eager scratch buffer of a stream
PyObject* py_set_scratch(PyObject*, PyObject* args) {
  PyObject* cap;
  int device = 0;
  unsigned long long stream = 0, ptr = 0;
  long long bytes = 0;
  if (!PyArg_ParseTuple(args, "OiKKL", &cap, &device, &stream, &ptr, &bytes)) return nullptr;
  State* s = state_of(cap);
  if (!s) return nullptr;
  s->sc_device = device;
  s->sc_stream = reinterpret_cast<void*>(static_cast<uintptr_t>(stream));
  s->sc_ptr = reinterpret_cast<void*>(static_cast<uintptr_t>(ptr));
  s->sc_bytes = bytes;
  Py_RETURN_NONE;
}

// The call itself.  Returns 0 (enqueued), a negative code of the library (the caller raises with
// the library's message), or kNotHandled.
long call(State* s, PyObject* y_slices, PyObject* x_obj, PyObject* a_list, PyObject* b_list, PyObject* indices, PyObject* metadata,
          double scaling, PyObject* y_packed, PyObject* eff_obj) {
  if (metadata == Py_None || !THPVariable_Check(x_obj)) return kNotHandled;
  if (!(PyList_Check(y_slices) || PyTuple_Check(y_slices)) || !(PyList_Check(a_list) || PyTuple_Check(a_list)) ||
      !(PyList_Check(b_list) || PyTuple_Check(b_list)))
    return kNotHandled;
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(y_slices);
  if (n < 1 || n > MLORA_MAX_SLICES || PySequence_Fast_GET_SIZE(a_list) != n || PySequence_Fast_GET_SIZE(b_list) != n) return kNotHandled;
  PyObject* target_obj = y_packed != Py_None ? y_packed : (n == 1 ? PySequence_Fast_GET_ITEM(y_slices, 0) : nullptr);
  if (!target_obj || !THPVariable_Check(target_obj)) return kNotHandled;

  std::string key;
  const at::Tensor* a0 = nullptr;
  if (!weights_key(a_list, b_list, n, &key, &a0)) return kNotHandled;
  const auto it = s->sites.find(key);
  if (it == s->sites.end()) return kNotHandled;
  const Site& site = it->second;
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* o = PySequence_Fast_GET_ITEM(y_slices, i);
    if (!THPVariable_Check(o)) return kNotHandled;
    const at::Tensor& y = THPVariable_Unpack(o);
    if (y.dim() < 1 || y.size(-1) != site.widths[static_cast<size_t>(i)]) return kNotHandled;
  }

  const at::Tensor& x = THPVariable_Unpack(x_obj);
  const at::Tensor& target = THPVariable_Unpack(target_obj);
  if (x.dim() != 2 || x.stride(1) != 1 || target.dim() != 2 || target.stride(1) != 1) return kNotHandled;
  const int64_t rows = x.size(0);
  if (rows <= 0 || rows > INT32_MAX) return kNotHandled;

  // the flag and the slot vector of the step's metadata (attribute reads: the object is the engine's)
  PyObject* flag = PyObject_GetAttrString(metadata, "no_lora_flag");
  if (!flag) { PyErr_Clear(); return kNotHandled; }
  const int no_lora = PyObject_IsTrue(flag);
  Py_DECREF(flag);
  if (no_lora != 0) { PyErr_Clear(); return kNotHandled; }
  const Ref tts{PyObject_GetAttrString(metadata, "token_to_slot")};
  if (!tts.p) { PyErr_Clear(); return kNotHandled; }
  PyObject* source_obj = tts.p != Py_None ? tts.p : indices;
  if (!THPVariable_Check(source_obj)) return kNotHandled;
  const at::Tensor& source = THPVariable_Unpack(source_obj);

  const int dev = site.device;
  if (x.size(1) != site.k || x.scalar_type() != site.dtype || target.scalar_type() != site.dtype || !on_device(x, dev) ||
      !on_device(target, dev) || !on_device(source, dev) || source.numel() < rows || target.size(0) < rows ||
      source.scalar_type() != c10::ScalarType::Int || source.dim() != 1 || !source.is_contiguous())
    return kNotHandled;
  const void* eff_ptr = nullptr;
  if (eff_obj != Py_None) {
    if (!THPVariable_Check(eff_obj)) return kNotHandled;
    const at::Tensor& eff = THPVariable_Unpack(eff_obj);
    if (eff.scalar_type() != c10::ScalarType::Int || !eff.is_contiguous() || eff.numel() < site.num_slots || !on_device(eff, dev)) return kNotHandled;
    eff_ptr = eff.data_ptr();
  }
  if (c10::hip::current_device() != dev) return kNotHandled;  // another GPU of this process: the Python path makes it current
  hipStream_t stream = c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(dev)).stream();

  const void* x_ptr = x.data_ptr();
  void* y_ptr = target.data_ptr();
  const int64_t xs = x.stride(0), ys = target.stride(0);
  const void* plan = nullptr;
  void* ws = nullptr;
  int64_t ws_bytes = 0;
  if (site.vectorisable && site.form != MLORA_FORM_TOKEN &&
      !(xs % 8 || ys % 8 || reinterpret_cast<uintptr_t>(x_ptr) % 16 || reinterpret_cast<uintptr_t>(y_ptr) % 16)) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) { (void)hipGetLastError(); return kNotHandled; }
    if (capturing != hipStreamCaptureStatusNone) return kNotHandled;
    uint32_t version = 0;
    try {
      version = source._version();
    } catch (...) {  // inference tensors carry no version counter: nothing is remembered for them
      return kNotHandled;
    }
    if (s->metadata != metadata || s->source != source_obj || s->version != version || s->stream != stream || s->num_slots != site.num_slots ||
        s->rows != rows || !s->plan)
      return kNotHandled;
    plan = s->plan;
    const uint64_t shape = (static_cast<uint64_t>(rows) << 24) | (static_cast<uint64_t>(site.num_slices) << 16) |
                           (static_cast<uint64_t>(site.rank) << 4) | static_cast<uint64_t>(site.dtype_code);
    int64_t need;
    const auto nit = s->need.find(shape);
    if (nit != s->need.end()) {
      need = nit->second;
    } else {
      if (s->need.size() >= 256) s->need.clear();
      need = static_cast<int64_t>(s->workspace_bytes(static_cast<int32_t>(rows), site.num_slices, site.rank, site.dtype_code));
      s->need.emplace(shape, need);
    }
    if (s->sc_device != dev || s->sc_stream != stream || !s->sc_ptr || s->sc_bytes < need) return kNotHandled;
    ws = s->sc_ptr;
    ws_bytes = s->sc_bytes;
  }

  MloraAddArgs* a = site.args;
  a->stream = stream;
  a->x = x_ptr;
  a->y = y_ptr;
  a->x_stride = xs;
  a->y_stride = ys;
  a->token_to_slot = static_cast<const int32_t*>(source.data_ptr());
  a->plan = static_cast<const int32_t*>(plan);
  a->num_tokens = static_cast<int32_t>(rows);
  a->scaling = static_cast<float>(scaling);
  a->workspace = ws;
  a->workspace_bytes = ws_bytes;
  a->effective_rank = static_cast<const int32_t*>(eff_ptr);
  return s->add_lora(a);
}

// call(state, y_slices, x, lora_a_slices, lora_b_slices, indices, metadata, scaling, y_packed, effective_rank)
PyObject* py_call(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs != 10) {
    PyErr_SetString(PyExc_TypeError, "call() takes ten arguments");
    return nullptr;
  }
  State* s = state_of(args[0]);
  if (!s) return nullptr;
  const double scaling = PyFloat_AsDouble(args[7]);
  if (scaling == -1.0 && PyErr_Occurred()) { PyErr_Clear(); return PyLong_FromLong(kNotHandled); }
  long rc;
  try {
    rc = call(s, args[1], args[2], args[3], args[4], args[5], args[6], scaling, args[8], args[9]);
  } catch (...) {  // whatever a tensor accessor objects to: the Python path says it in its own words
    rc = kNotHandled;
  }
  if (PyErr_Occurred()) PyErr_Clear();
  if (rc == kNotHandled) ++s->passed_on;
  else ++s->handled;
  return PyLong_FromLong(rc);
}

PyObject* py_counters(PyObject*, PyObject* cap) {
  State* s = state_of(cap);
  if (!s) return nullptr;
  return Py_BuildValue("(LL)", s->handled, s->passed_on);
}

PyMethodDef kMethods[] = {
    {"create", py_create, METH_VARARGS, "create(address of mlora_add_lora, address of mlora_add_workspace_bytes) -> state"},
    {"register_site", py_register_site, METH_VARARGS, "register_site(state, a_list, b_list, widths, block address, block owner, vectorisable) -> bool"},
    {"clear_sites", py_clear_sites, METH_O, "clear_sites(state)"},
    {"set_step", py_set_step, METH_VARARGS, "set_step(state, metadata, source, version, stream, num_slots, rows, plan address)"},
    {"forget_step", py_forget_step, METH_O, "forget_step(state)"},
    {"set_scratch", py_set_scratch, METH_VARARGS, "set_scratch(state, device index, stream, address, bytes)"},
    {"counters", py_counters, METH_O, "counters(state) -> (calls enqueued here, calls left to the Python path)"},
    {"call", reinterpret_cast<PyCFunction>(reinterpret_cast<void (*)()>(py_call)), METH_FASTCALL,
     "call(state, y_slices, x, lora_a_slices, lora_b_slices, indices, metadata, scaling, y_packed, effective_rank) -> 0, a library error code, or NOT_HANDLED"},
    {nullptr, nullptr, 0, nullptr},
};

PyModuleDef kModule = {PyModuleDef_HEAD_INIT, "_mlora_fastcall", "C++ host path of the usual add_lora call", -1, kMethods, nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__mlora_fastcall(void) {
  PyObject* m = PyModule_Create(&kModule);
  if (m) PyModule_AddIntConstant(m, "NOT_HANDLED", kNotHandled);
  return m;
}
