// Fixed pool of recurrent-state slots: one slot per live sequence of a model that carries per-sequence state next to
// (or instead of) paged KV (token-shift rows, short-convolution tails, state-space matrices). A slot names one row
// of every such state tensor. Slots are handed out lowest-first, so a freed slot is the next one reused; the kernels
// treat a sequence that starts at position 0 as having zero state, so a reused slot needs no clearing.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstdint>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>

namespace py = pybind11;

namespace kafka {

class StateSlots {
 public:
  explicit StateSlots(int n) : n_(n) {
    if (n < 1) throw std::invalid_argument("StateSlots: at least one slot");
    for (int i = 0; i < n; ++i) free_.insert(i);
  }
  int num_slots() const { return n_; }
  int num_free() const { return (int)free_.size(); }
  bool has(int64_t sid) const { return owner_.count(sid) != 0; }
  // -1 when the pool is dry (the caller defers the admission)
  int acquire(int64_t sid) {
    auto it = owner_.find(sid);
    if (it != owner_.end()) return it->second;
    if (free_.empty()) return -1;
    const int s = *free_.begin();
    free_.erase(free_.begin());
    owner_[sid] = s;
    ++acquired_;
    return s;
  }
  void release(int64_t sid) {
    auto it = owner_.find(sid);
    if (it == owner_.end()) return;
    free_.insert(it->second);
    owner_.erase(it);
  }
  int slot_of(int64_t sid) const {
    auto it = owner_.find(sid);
    if (it == owner_.end()) throw std::runtime_error("no state slot for sequence " + std::to_string(sid));
    return it->second;
  }
  py::dict stats() const {
    py::dict d;
    d["slots"] = n_;
    d["free"] = (int)free_.size();
    d["acquired_total"] = acquired_;
    return d;
  }

 private:
  int n_;
  int64_t acquired_ = 0;
  std::set<int> free_;
  std::unordered_map<int64_t, int> owner_;
};

void register_state_slots(py::module& m) {
  py::class_<StateSlots>(m, "StateSlots")
      .def(py::init<int>(), py::arg("num_slots"))
      .def_property_readonly("num_slots", &StateSlots::num_slots)
      .def("num_free", &StateSlots::num_free)
      .def("has", &StateSlots::has)
      .def("acquire", &StateSlots::acquire)
      .def("release", &StateSlots::release)
      .def("slot_of", &StateSlots::slot_of)
      .def("stats", &StateSlots::stats);
}

}  // namespace kafka
