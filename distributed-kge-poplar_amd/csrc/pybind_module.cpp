// Python module `libpoplar_kge`: the reference's low-level interface
// (src/lib.cpp:38-52: Engine(settings, gp_folder) and Engine.run(command, data))
// bound onto the C-ABI of include/kge_hip.h.  A settings / data dict holds str,
// bool, int, float, dict[str, float] and C-contiguous numpy arrays of float32,
// uint32 or int16 (float16 bits, as the reference passes them, src/lib.cpp:25-35).
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <deque>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/kge_hip.h"

namespace py = pybind11;

namespace {

// Owns the storage a kge_item array points into for the duration of a call.
struct ItemPack {
    std::vector<kge_item> items;
    std::deque<std::string> strings;
    std::deque<std::vector<size_t>> shapes;
    std::deque<std::vector<const char*>> map_keys;
    std::deque<std::vector<float>> map_vals;
    std::vector<py::object> keep;

    explicit ItemPack(const py::dict& d) {
        items.reserve(d.size());
        for (auto kv : d) {
            kge_item it = {};
            strings.push_back(py::cast<std::string>(kv.first));
            it.key = strings.back().c_str();
            const py::handle v = kv.second;
            if (py::isinstance<py::str>(v)) {
                it.kind = KGE_STR;
                strings.push_back(py::cast<std::string>(v));
                it.str = strings.back().c_str();
            } else if (py::isinstance<py::array>(v)) {
                py::array a = py::reinterpret_borrow<py::array>(v);
                const py::dtype dt = a.dtype();
                if (dt.is(py::dtype::of<float>())) it.kind = KGE_F32;
                else if (dt.is(py::dtype::of<uint32_t>())) it.kind = KGE_U32;
                else if (dt.is(py::dtype::of<int16_t>()) || (dt.kind() == 'f' && dt.itemsize() == 2)) it.kind = KGE_F16;
                else
                    throw std::invalid_argument("Key '" + strings.back() +
                                                "': arrays must be float32, uint32 or int16 (float16 bits)");
                if (!(a.flags() & py::array::c_style))
                    throw std::invalid_argument("Key '" + strings.back() + "': array must be C-contiguous");
                shapes.emplace_back(a.shape(), a.shape() + a.ndim());
                it.shape = shapes.back().data();
                it.rank = shapes.back().size();
                it.data = const_cast<void*>(a.data());
                keep.push_back(a);
            } else if (py::isinstance<py::bool_>(v)) {
                it.kind = KGE_BOOL;
                it.num = py::cast<bool>(v) ? 1.0 : 0.0;
            } else if (py::isinstance<py::int_>(v) || py::hasattr(v, "__index__")) {
                it.kind = KGE_UINT;
                const long long x = py::cast<long long>(v);
                if (x < 0 || x > 0xffffffffLL)
                    throw std::invalid_argument("Key '" + strings.back() + "': integer out of unsigned range");
                it.num = (double)x;
            } else if (py::isinstance<py::float_>(v) || py::hasattr(v, "__float__")) {
                it.kind = KGE_FLOAT;
                it.num = py::cast<double>(v);
            } else if (py::isinstance<py::dict>(v)) {
                it.kind = KGE_MAP;
                map_keys.emplace_back();
                map_vals.emplace_back();
                for (auto mk : py::reinterpret_borrow<py::dict>(v)) {
                    strings.push_back(py::cast<std::string>(mk.first));
                    map_keys.back().push_back(strings.back().c_str());
                    map_vals.back().push_back(py::cast<float>(mk.second));
                }
                it.map_keys = map_keys.back().data();
                it.map_vals = map_vals.back().data();
                it.map_len = map_keys.back().size();
            } else {
                throw std::invalid_argument("Key '" + strings.back() + "' holds a value of unsupported type " +
                                            py::cast<std::string>(py::str(py::type::of(v))));
            }
            items.push_back(it);
        }
    }
};

[[noreturn]] void raise(int status, const char* msg) {
    if (status == KGE_INVALID_ARGUMENT) throw std::invalid_argument(msg);  // -> ValueError
    if (status == KGE_LOGIC_ERROR) throw std::logic_error(msg);
    throw std::runtime_error(msg);                                         // -> RuntimeError
}

class Engine {
   public:
    Engine(const py::dict& settings, const std::string& gp_folder) {
        ItemPack pack(settings);
        char err[1024] = {0};
        const int rc = kge_engine_create(pack.items.data(), pack.items.size(), gp_folder.c_str(), &engine_,
                                         err, sizeof(err));
        if (rc != KGE_OK) raise(rc, err);
    }
    ~Engine() { kge_engine_destroy(engine_); }
    Engine(const Engine&) = delete;
    Engine& operator=(const Engine&) = delete;

    py::dict run(const std::string& command, const py::dict& data) {
        py::dict result;
        if (command == "variables") {
            py::list vars;
            for (size_t i = 0; i < kge_engine_variable_count(engine_); ++i) {
                const char* name;
                const size_t* shape;
                size_t rank;
                kge_engine_variable_info(engine_, i, &name, &shape, &rank);
                vars.append(py::make_tuple(std::string(name), std::vector<unsigned>(shape, shape + rank)));
            }
            result["variables"] = vars;
            return result;
        }
        ItemPack pack(data);
        char err[1024] = {0};
        int rc;
        {
            // the reference holds the GIL for the whole call (src/lib.cpp:50); so do we
            rc = kge_engine_run(engine_, command.c_str(), pack.items.data(), pack.items.size(), err, sizeof(err));
        }
        if (rc != KGE_OK) raise(rc, err);
        return result;
    }

   private:
    kge_engine* engine_ = nullptr;
};

}  // namespace

PYBIND11_MODULE(libpoplar_kge, m) {
    m.doc() = "Low-level interface of the MI355X KGE training step (use the poplar_kge Python wrapper)";
    py::class_<Engine>(m, "Engine", "Allocate the tables on the HIP device and prepare the step")
        .def(py::init<const py::dict&, const std::string&>(), py::arg("settings"), py::arg("gp_folder"))
        .def("run", &Engine::run, "Execute a command (see Python for usage)", py::arg("command"),
             py::arg("data"));
}
