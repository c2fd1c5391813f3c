// Host runtime of the engine, in C++: page and slot pools, the cache manager (groups of layers,
// block tables, windows), the builder of a step's int32 buffer (tokens, positions, per-request row
// ranges, write addresses, block tables, attention work lists) in cache.hpp, and the scheduler's
// mechanics in scheduler.hpp.
//
// Role in the reference: PageAllocator / PagedTable / page_offsets
// (crates/mach-model/src/paged_kv.rs:18-68, 229-289) and the per-step staging of
// decode_step_explicit (crates/mach-model/src/batched.rs:2914-3038, 4799-4817), which are Rust.
// Python binds these classes with pybind11; policy that is not on the per-step path (which
// architecture, which parts, finish reasons) stays in Python.
#include "scheduler.hpp"

using namespace mshost;

PYBIND11_MODULE(ms_host, m) {
    m.doc() = "machserve_amd host runtime: pools, cache manager, step buffer builder";
    // translators are tried newest first, so the derived class is registered last
    auto& cache_error = py::register_exception<CacheError>(m, "CacheError", PyExc_RuntimeError);
    py::register_exception<OutOfPages>(m, "OutOfPages", cache_error.ptr());
    py::class_<BlockPool>(m, "BlockPool")
        .def(py::init<int>())
        .def_property_readonly("num_pages", &BlockPool::num_pages)
        .def("available", &BlockPool::available)
        .def("alloc", [](BlockPool& p) -> py::object { int r = p.alloc(); return r < 0 ? py::none() : py::object(py::int_(r)); })
        .def("free", &BlockPool::free)
        .def("live_pages", &BlockPool::live_pages);
    py::class_<SlotPool>(m, "SlotPool")
        .def(py::init<int>())
        .def_property_readonly("num_slots", &SlotPool::num_slots)
        .def("available", &SlotPool::available)
        .def("alloc", [](SlotPool& p) -> py::object { int r = p.alloc(); return r < 0 ? py::none() : py::object(py::int_(r)); })
        .def("free", &SlotPool::free)
        .def("is_live", &SlotPool::is_live);
    py::class_<CacheCore>(m, "CacheCore")
        .def(py::init<int, int>())
        .def("add_group", &CacheCore::add_group)
        .def_property_readonly("page_size", &CacheCore::page_size)
        .def_property_readonly("max_requests", &CacheCore::max_requests)
        .def("num_groups", &CacheCore::num_groups)
        .def("group_name", &CacheCore::group_name)
        .def("group_window", &CacheCore::group_window)
        .def("group_pages", &CacheCore::group_pages)
        .def("group_available", &CacheCore::group_available)
        .def("group_live_pages", &CacheCore::group_live_pages)
        .def("scratch_page", &CacheCore::scratch_page)
        .def("scratch_slot", &CacheCore::scratch_slot)
        .def("slots_available", &CacheCore::slots_available)
        .def("slot_is_live", &CacheCore::slot_is_live)
        .def("admit", &CacheCore::admit)
        .def("length", &CacheCore::length)
        .def("lengths", &CacheCore::lengths)
        .def("pages_needed", &CacheCore::pages_needed)
        .def("can_extend", &CacheCore::can_extend)
        .def("extend", &CacheCore::extend)
        .def("commit", &CacheCore::commit)
        .def("release", &CacheCore::release)
        .def("table", &CacheCore::table)
        .def("slot_of_position", &CacheCore::slot_of_position)
        .def("live_requests", &CacheCore::live_requests)
        .def("check", &CacheCore::check)
        .def("build_step", &CacheCore::build_step, py::arg("slots"), py::arg("counts"), py::arg("tokens"), py::arg("want_rows"),
             py::arg("heads_per_kv"), py::arg("rows_per_block"), py::arg("table_multiple") = 1, py::arg("pad_rows") = 0, py::arg("axes") = 1,
             py::arg("explicit_positions") = std::vector<int>(), py::arg("fill_rows") = 0, py::arg("fill_seqs") = 0,
             py::arg("fill_want") = 0);

    py::register_exception<SchedulerError>(m, "SchedulerError", PyExc_ValueError);
    py::class_<PlanItem>(m, "PlanItem")
        .def_readonly("id", &PlanItem::id)
        .def_readonly("start", &PlanItem::start)
        .def_readonly("count", &PlanItem::count)
        .def_readonly("sample", &PlanItem::sample);
    py::class_<StepPlan>(m, "StepPlan")
        .def_readonly("items", &StepPlan::items)
        .def_readonly("preempted", &StepPlan::preempted)
        .def_readonly("admitted", &StepPlan::admitted);
    py::class_<SchedulerCore>(m, "SchedulerCore")
        .def(py::init<CacheCore&, int, int, int, int>(), py::keep_alive<1, 2>())
        .def_property_readonly("max_batch_tokens", &SchedulerCore::max_batch_tokens)
        .def_property_readonly("chunk_size", &SchedulerCore::chunk_size)
        .def_property_readonly("max_running", &SchedulerCore::max_running)
        .def("add", &SchedulerCore::add)
        .def("has_work", &SchedulerCore::has_work)
        .def("waiting", &SchedulerCore::waiting)
        .def("running", &SchedulerCore::running)
        .def("fed", &SchedulerCore::fed)
        .def("slot", &SchedulerCore::slot)
        .def("decoding", &SchedulerCore::decoding)
        .def("schedule", &SchedulerCore::schedule)
        .def("advance", &SchedulerCore::advance)
        .def("finish", &SchedulerCore::finish);
}
