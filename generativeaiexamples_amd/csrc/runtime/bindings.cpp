// pybind11 module `generativeaiexamples_amd._rt`: the native host runtime.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>

#include "block_manager.h"
#include "grammar.h"
#include "scheduler.h"
#include "shm_channel.h"

namespace py = pybind11;
using namespace gai;

// compiled schema node (engine/guided.py) -> GNode
static GNode gnode_from(const py::dict& d) {
  GNode n;
  n.kind = d["kind"].cast<int>();
  auto get_i = [&](const char* k, int dflt) { return d.contains(k) ? d[k].cast<int>() : dflt; };
  n.item = get_i("item", -1);
  n.min_items = get_i("min_items", 0);
  n.max_items = get_i("max_items", 1 << 20);
  n.min_len = get_i("min_len", 0);
  n.max_len = get_i("max_len", 256);
  n.disc_prop = get_i("disc_prop", -1);
  n.dep_prop = get_i("dep_prop", -1);
  if (d.contains("keys")) n.keys = d["keys"].cast<std::vector<std::string>>();
  if (d.contains("props")) n.props = d["props"].cast<std::vector<int>>();
  if (d.contains("required")) {
    for (bool r : d["required"].cast<std::vector<bool>>()) n.required.push_back(r ? 1 : 0);
  }
  if (d.contains("dep_alts")) n.dep_alts = d["dep_alts"].cast<std::vector<int>>();
  if (d.contains("lits")) n.lits = d["lits"].cast<std::vector<std::string>>();
  if (d.contains("alts")) n.alts = d["alts"].cast<std::vector<int>>();
  n.required.resize(n.props.size(), 1);
  if (n.keys.size() != n.props.size()) throw std::invalid_argument("grammar node: keys/props size mismatch");
  return n;
}

template <typename T>
py::array_t<T> arr(const std::vector<T>& v) {
  py::array_t<T> a(v.size());
  if (!v.empty()) std::memcpy(a.mutable_data(), v.data(), v.size() * sizeof(T));
  return a;
}

template <typename T>
py::array_t<T> arr2(const std::vector<T>& v, int cols) {
  const size_t rows = cols ? v.size() / cols : 0;
  py::array_t<T> a({rows, (size_t)cols});
  if (!v.empty()) std::memcpy(a.mutable_data(), v.data(), v.size() * sizeof(T));
  return a;
}

PYBIND11_MODULE(_rt, m) {
  m.doc() = "native host runtime: paged-KV block manager + continuous-batching scheduler";
  m.attr("BLOCK_SIZE") = kBlockSize;

  py::class_<BlockManager>(m, "BlockManager")
      .def(py::init<int, bool>(), py::arg("num_blocks"), py::arg("prefix_cache") = true)
      .def("alloc", &BlockManager::alloc)
      .def("incref", &BlockManager::incref)
      .def("decref", &BlockManager::decref)
      .def("num_free", &BlockManager::num_free)
      .def("num_blocks", &BlockManager::num_blocks)
      .def("can_allocate", &BlockManager::can_allocate)
      .def("match_prefix", &BlockManager::match_prefix)
      .def("commit", &BlockManager::commit)
      .def_static("chain_hash",
                  [](uint64_t parent, const std::vector<int>& t) {
                    return BlockManager::chain_hash(parent, t.data(), (int)t.size());
                  });

  py::class_<StepBatch>(m, "StepBatch")
      .def_property_readonly("token_ids", [](const StepBatch& b) { return arr(b.token_ids); })
      .def_property_readonly("positions", [](const StepBatch& b) { return arr(b.positions); })
      .def_property_readonly("slots", [](const StepBatch& b) { return arr(b.slots); })
      .def_property_readonly("prefill_seq_ids", [](const StepBatch& b) { return b.prefill_seq_ids; })
      .def_property_readonly("cu_q", [](const StepBatch& b) { return arr(b.cu_q); })
      .def_property_readonly("prefill_ctx", [](const StepBatch& b) { return arr(b.prefill_ctx); })
      .def_property_readonly("prefill_qlen", [](const StepBatch& b) { return b.prefill_qlen; })
      .def_property_readonly("prefill_block_tables",
                             [](const StepBatch& b) { return arr2(b.prefill_block_tables, b.max_blocks); })
      .def_property_readonly("prefill_samples",
                             [](const StepBatch& b) { return std::vector<int>(b.prefill_samples.begin(), b.prefill_samples.end()); })
      .def_property_readonly("decode_seq_ids", [](const StepBatch& b) { return b.decode_seq_ids; })
      .def_property_readonly("decode_ctx", [](const StepBatch& b) { return arr(b.decode_ctx); })
      .def_property_readonly("decode_block_tables",
                             [](const StepBatch& b) { return arr2(b.decode_block_tables, b.max_blocks); })
      .def_property_readonly("preempted", [](const StepBatch& b) { return b.preempted; })
      .def_readonly("max_blocks", &StepBatch::max_blocks)
      .def_readonly("num_prefill_tokens", &StepBatch::num_prefill_tokens)
      .def_property_readonly("num_tokens", [](const StepBatch& b) { return (int)b.token_ids.size(); });

  py::class_<Scheduler>(m, "Scheduler")
      .def(py::init<int, int, int, int, bool, int>(), py::arg("num_blocks"), py::arg("max_num_seqs"),
           py::arg("max_batched_tokens"), py::arg("max_model_len"), py::arg("prefix_cache") = true,
           py::arg("prefill_chunk") = 0)
      .def("add", &Scheduler::add, py::arg("id"), py::arg("prompt"), py::arg("max_new_tokens"),
           py::arg("priority") = 0)
      .def("abort", &Scheduler::abort)
      .def("finish", &Scheduler::finish)
      .def("append_tokens", &Scheduler::append_tokens)
      .def("schedule", &Scheduler::schedule, py::call_guard<py::gil_scoped_release>())
      .def("extend", &Scheduler::extend, py::arg("id"), py::arg("tokens"))
      .def("schedule_exact", &Scheduler::schedule_exact, py::arg("ids"), py::arg("counts"))
      .def("reserve_decode",
           [](Scheduler& s, const std::vector<int64_t>& ids, int steps) -> py::object {
             std::vector<int32_t> bt;
             int mb = 0;
             if (!s.reserve_decode(ids, steps, bt, mb)) return py::none();
             return arr2(bt, mb);
           },
           py::arg("ids"), py::arg("steps"),
           "reserve KV pages for a multi-step decode run; [len(ids), max_blocks] int32 block tables or None")
      .def("reserve_upto",
           [](Scheduler& s, const std::vector<int64_t>& ids, const std::vector<int>& upto) -> py::object {
             std::vector<int32_t> bt;
             int mb = 0;
             if (!s.reserve_upto(ids, upto, bt, mb)) return py::none();
             return arr2(bt, mb);
           },
           py::arg("ids"), py::arg("upto"),
           "own the KV pages of the first upto[i] positions of each sequence; block tables or None")
      .def("advance_decode", &Scheduler::advance_decode, py::arg("ids"), py::arg("toks"), py::arg("steps"),
           py::arg("chained") = false)
      .def("num_waiting", &Scheduler::num_waiting)
      .def("num_running", &Scheduler::num_running)
      .def("num_free_blocks", &Scheduler::num_free_blocks)
      .def("num_blocks", &Scheduler::num_blocks)
      .def("prefix_hit_rate", &Scheduler::prefix_hit_rate)
      .def("has_work", &Scheduler::has_work)
      .def("num_tokens", &Scheduler::num_tokens)
      .def("num_generated", &Scheduler::num_generated);

  py::class_<Grammar>(m, "Grammar")
      .def(py::init([](const py::list& nodes, int root, const py::list& vocab, std::vector<int> eos) {
             std::vector<GNode> ns;
             for (auto& o : nodes) ns.push_back(gnode_from(o.cast<py::dict>()));
             if (root < 0 || root >= (int)ns.size()) throw std::invalid_argument("grammar: bad root");
             std::vector<std::string> vb;
             vb.reserve(vocab.size());
             for (auto& o : vocab) vb.push_back(o.is_none() ? std::string() : o.cast<std::string>());
             return new Grammar(std::move(ns), root, vb, std::move(eos));
           }),
           py::arg("nodes"), py::arg("root"), py::arg("vocab"), py::arg("eos"),
           "nodes: compiled schema (list of dicts); vocab: bytes of every token id (None = never allowed)")
      .def_property_readonly("vocab_size", &Grammar::vocab_size)
      .def_property_readonly("max_token_len", &Grammar::max_token_len)
      .def("minlen", &Grammar::minlen);

  py::class_<Matcher>(m, "Matcher")
      .def(py::init<const Grammar*>(), py::arg("grammar"), py::keep_alive<1, 2>())
      .def("fill_mask",
           [](Matcher& mt, int budget, py::array_t<uint32_t, py::array::c_style> out) {
             if (out.size() * 32 < mt.vocab_size()) throw std::invalid_argument("fill_mask: mask too small");
             uint32_t* p = out.mutable_data();  // with the GIL held
             py::gil_scoped_release nogil;
             mt.fill_mask(budget, p);
           },
           py::arg("budget"), py::arg("out"),
           "allowed-token bitmask (uint32 words) for the next token, `budget` tokens left including it")
      .def("advance", &Matcher::advance, py::arg("token"))
      .def("feed_bytes", [](Matcher& mt, py::bytes b) { return mt.feed_bytes(std::string(b)); })
      .def_property_readonly("done", &Matcher::done)
      .def_property_readonly("dead", &Matcher::dead)
      .def_property_readonly("can_finish", &Matcher::can_finish)
      .def_property_readonly("min_chars", &Matcher::min_chars)
      .def_property_readonly("cache_size", &Matcher::cache_size);

  py::class_<ShmChannel>(m, "ShmChannel")
      .def_static("create", &ShmChannel::create, py::arg("name"), py::arg("num_readers"),
                  py::arg("slot_bytes") = 8 << 20, py::arg("num_slots") = 4, py::return_value_policy::take_ownership)
      .def_static("open", &ShmChannel::open, py::arg("name"), py::arg("reader"), py::arg("timeout_s") = 60.0,
                  py::call_guard<py::gil_scoped_release>(), py::return_value_policy::take_ownership)
      .def("send",
           [](ShmChannel& c, py::bytes msg, double timeout_s) {
             char* buf = nullptr;
             Py_ssize_t len = 0;
             if (PyBytes_AsStringAndSize(msg.ptr(), &buf, &len) != 0) throw py::error_already_set();
             bool ok;
             {
               py::gil_scoped_release nogil;
               ok = c.send(buf, (uint64_t)len, timeout_s);
             }
             return ok;
           },
           py::arg("msg"), py::arg("timeout_s") = -1.0,
           "publish one message to every reader; False if a reader did not free a slot within timeout_s")
      .def("recv",
           [](ShmChannel& c, double timeout_s) -> py::object {
             std::vector<char> out;
             int rc;
             {
               py::gil_scoped_release nogil;
               rc = c.recv(out, timeout_s);
             }
             if (rc == 1) return py::none();
             if (rc == 2) throw std::runtime_error("ShmChannel: the writer process is gone");
             return py::bytes(out.data(), out.size());
           },
           py::arg("timeout_s") = -1.0, "next message (bytes), or None on timeout")
      .def_property_readonly("slot_bytes", &ShmChannel::slot_bytes)
      .def_property_readonly("num_readers", &ShmChannel::num_readers)
      .def_property_readonly("sent", &ShmChannel::sent);
}
