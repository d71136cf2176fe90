// TorchScript custom class `torch.classes.vesin._NeighborList` on top of this library's C ABI.
//
// Same registered name, constructor, `compute` signature, pickle keys and error texts as the reference's class
// (vesin-torch/src/vesin_torch.cpp:52-321, vesin-torch/include/vesin_torch.hpp:36-108), so that a scripted or
// exported model that holds the reference's class loads this one instead. Differences, all on the device side:
//   - pairs are handed out as int64 views of the size_t arrays the kernels wrote (every index is below 2^63, so
//     the bits are the same): no conversion pass over 16 bytes per pair (the reference converts, :225-226);
//   - the kernels run on the caller's current stream (vesin_hip_neighbors_on_stream), ordered after whatever
//     produced the inputs there, instead of on the null stream;
//   - with `copy=true` (the default) the rows are not copied out of the list's arrays (the reference clones every
//     array, :214-256): the list takes its arrays from PyTorch's caching allocator (vesin_hip_set_output_allocator)
//     and the tensors that go to the caller take them over (vesin_hip_detach_outputs), the next call gets new ones
//     from the allocator's cache. Arrays much larger than their rows are copied as before.
// The gradient of distances and vectors with respect to points and box (reference :403-479) is one HIP kernel
// of the library (vesin_hip_pairs_backward) instead of a chain of tensor operations.

#include <cstdlib>
#include <cstring>
#include <sstream>
#include <string>
#include <vector>

#include <torch/torch.h>

#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPStream.h>

#include "vesin.h"

// What vesin_hip_set_output_allocator is given: device memory from PyTorch's caching allocator (of the current
// device, for the current stream, like the memory of any tensor made now). Exported for callers that bind the C ABI
// themselves (the ctypes caller of this package passes their addresses on).
extern "C" __attribute__((visibility("default"))) void* vesin_amd_torch_allocate(size_t bytes, void* /*context*/) {
    try {
        return c10::hip::HIPCachingAllocator::raw_alloc(bytes);
    } catch (...) {
        return nullptr; // (the library reports "failed to allocate memory")
    }
}

extern "C" __attribute__((visibility("default"))) void vesin_amd_torch_release(void* pointer, void* /*context*/) {
    try {
        c10::hip::HIPCachingAllocator::raw_delete(pointer);
    } catch (...) {
    }
}

namespace vesin_amd_torch {

/// A tensor over `rows` rows at the start of an array that came from vesin_amd_torch_allocate; the array goes back to
/// the allocator with the tensor's storage.
static torch::Tensor adopt_array(void* data, std::vector<int64_t> shape, torch::ScalarType dtype, const torch::Device& device) {
    return torch::from_blob(
        data, shape, [](void* pointer) { vesin_amd_torch_release(pointer, nullptr); },
        torch::TensorOptions().device(device).dtype(dtype)
    );
}

/// The same for callers outside of this file (`torch.ops.vesin_amd.adopt`).
static torch::Tensor adopt(int64_t pointer, std::vector<int64_t> shape, torch::ScalarType dtype, int64_t device_index) {
    return adopt_array(
        reinterpret_cast<void*>(static_cast<uintptr_t>(pointer)), std::move(shape), dtype,
        torch::Device(torch::kCUDA, static_cast<c10::DeviceIndex>(device_index))
    );
}

static VesinDevice to_vesin(const torch::Device& device) {
    if (device.is_cuda()) {
        // PyTorch-ROCm names HIP devices "cuda"
        return VesinDevice{VesinCUDA, static_cast<int>(device.index())};
    }
    if (device.is_cpu()) {
        return VesinDevice{VesinCPU, 0};
    }
    throw std::runtime_error("device " + device.str() + " is not supported in vesin");
}

static VesinAlgorithm parse_algorithm(const std::string& name) {
    if (name == "auto") {
        return VesinAutoAlgorithm;
    }
    if (name == "brute_force") {
        return VesinBruteForce;
    }
    if (name == "cell_list") {
        return VesinCellList;
    }
    throw std::runtime_error(
        "unknown algorithm '" + name + "', expected one of 'auto', 'brute_force', or 'cell_list'"
    );
}

/// Gradient of the pair geometry: d(distances, vectors) / d(points, box). Pairs and shifts are constants.
class PairGeometry: public torch::autograd::Function<PairGeometry> {
public:
    static torch::autograd::variable_list forward(
        torch::autograd::AutogradContext* context,
        torch::Tensor points,
        torch::Tensor box,
        torch::Tensor pairs,
        torch::Tensor shifts,
        torch::Tensor distances,
        torch::Tensor vectors,
        bool any_periodic
    ) {
        context->save_for_backward({pairs, shifts, distances, vectors});
        context->saved_data["points_grad"] = points.requires_grad();
        context->saved_data["box_grad"] = box.requires_grad() && any_periodic;
        context->saved_data["n_points"] = points.size(0);
        return {distances, vectors};
    }

    static torch::autograd::variable_list backward(
        torch::autograd::AutogradContext* context,
        torch::autograd::variable_list grads
    ) {
        const auto saved = context->get_saved_variables();
        const auto& pairs = saved[0];
        const auto& shifts = saved[1];
        const auto& distances = saved[2];
        const auto& vectors = saved[3];
        const bool want_points = context->saved_data["points_grad"].toBool();
        const bool want_box = context->saved_data["box_grad"].toBool();
        const int64_t n_points = context->saved_data["n_points"].toInt();

        auto points_grad = torch::Tensor();
        auto box_grad = torch::Tensor();
        if (want_points || want_box) {
            const auto options = vectors.options();
            const int64_t n_pairs = pairs.size(0);
            auto distances_grad = grads[0].defined() ? grads[0].contiguous() : torch::Tensor();
            auto vectors_grad = grads[1].defined() ? grads[1].contiguous() : torch::Tensor();
            if (want_points) {
                points_grad = torch::zeros({n_points, 3}, options);
            }
            if (want_box) {
                box_grad = torch::zeros({3, 3}, options);
            }
            if (n_pairs > 0 && (distances_grad.defined() || vectors_grad.defined())) {
                TORCH_CHECK(vectors.is_cuda(), "the gradient of a neighbor list is computed on the GPU only");
                const char* error_message = nullptr;
                const auto status = vesin_hip_pairs_backward(
                    reinterpret_cast<const size_t (*)[2]>(pairs.data_ptr<int64_t>()),
                    want_box ? reinterpret_cast<const int32_t (*)[3]>(shifts.data_ptr<int32_t>()) : nullptr,
                    distances.data_ptr<double>(),
                    reinterpret_cast<const double (*)[3]>(vectors.data_ptr<double>()),
                    static_cast<size_t>(n_pairs),
                    distances_grad.defined() ? distances_grad.data_ptr<double>() : nullptr,
                    vectors_grad.defined() ? reinterpret_cast<const double (*)[3]>(vectors_grad.data_ptr<double>()) : nullptr,
                    static_cast<size_t>(n_points),
                    VesinDevice{VesinCUDA, static_cast<int>(vectors.device().index())},
                    want_points ? reinterpret_cast<double (*)[3]>(points_grad.data_ptr<double>()) : nullptr,
                    want_box ? reinterpret_cast<double (*)[3]>(box_grad.data_ptr<double>()) : nullptr,
                    current_stream(vectors.device()),
                    &error_message
                );
                if (status != EXIT_SUCCESS) {
                    throw std::runtime_error(std::string("failed to compute the gradient of neighbors: ") + error_message);
                }
            }
        }
        return {points_grad, box_grad, torch::Tensor(), torch::Tensor(), torch::Tensor(), torch::Tensor(), torch::Tensor()};
    }

    /// The stream PyTorch queues the caller's work on: the library's kernels go there too.
    static void* current_stream(const torch::Device& device) {
        return static_cast<void*>(c10::hip::getCurrentHIPStream(device.index()).stream());
    }
};

class NeighborListHolder: public torch::CustomClassHolder {
public:
    NeighborListHolder(double cutoff, bool full_list, bool sorted, std::string algorithm, int64_t n_threads):
        cutoff_(cutoff),
        full_list_(full_list),
        sorted_(sorted),
        algorithm_(std::move(algorithm)),
        n_threads_(n_threads) {
        if (n_threads_ < 0) {
            throw std::runtime_error("n_threads must be zero or a positive integer");
        }
    }

    ~NeighborListHolder() override {
        vesin_free(&list_);
    }

    NeighborListHolder(const NeighborListHolder&) = delete;
    NeighborListHolder& operator=(const NeighborListHolder&) = delete;

    std::vector<torch::Tensor> compute(
        torch::Tensor points,
        torch::Tensor box,
        torch::Tensor periodic,
        std::string quantities,
        bool copy
    ) {
        if (points.device() != box.device()) {
            C10_THROW_ERROR(
                ValueError,
                "expected `points` and `box` to have the same device, got " + points.device().str() + " and " +
                    box.device().str()
            );
        }
        const auto device = to_vesin(points.device());
        if (points.scalar_type() != box.scalar_type()) {
            C10_THROW_ERROR(
                ValueError,
                std::string("expected `points` and `box` to have the same dtype, got ") +
                    torch::toString(points.scalar_type()) + " and " + torch::toString(box.scalar_type())
            );
        }
        if (points.scalar_type() != torch::kFloat64) {
            C10_THROW_ERROR(ValueError, "only float64 is supported for `points` and `box`");
        }
        if (points.dim() != 2 || points.size(1) != 3) {
            std::ostringstream text;
            text << "`points` must be n x 3 tensor, but the shape is " << points.sizes();
            C10_THROW_ERROR(ValueError, text.str());
        }
        if (box.dim() != 2 || box.size(0) != 3 || box.size(1) != 3) {
            std::ostringstream text;
            text << "`box` must be 3 x 3 tensor, but the shape is " << box.sizes();
            C10_THROW_ERROR(ValueError, text.str());
        }
        if (periodic.scalar_type() != torch::kBool) {
            C10_THROW_ERROR(ValueError, "`periodic` must be a tensor of bool");
        }
        if (periodic.dim() == 0) {
            periodic = periodic.repeat({3});
        }
        if (periodic.dim() != 1 || periodic.size(0) != 3) {
            C10_THROW_ERROR(ValueError, "`periodic` must be either a single bool or a tensor of 3 bool");
        }
        for (const char letter : quantities) {
            if (std::strchr("ijPSdD", letter) == nullptr || letter == '\0') {
                C10_THROW_ERROR(ValueError, "unexpected character in `quantities`: " + std::string(1, letter));
            }
        }

        // which periodic directions there are is needed on the host only for the gradient of the box
        const bool differentiate = points.requires_grad() || box.requires_grad();
        bool any_periodic = true;
        if (box.requires_grad()) {
            any_periodic = periodic.any().item<bool>();
        }
        if (periodic.device() != points.device()) {
            periodic = periodic.to(points.device());
        }
        periodic = periodic.contiguous();

        const bool want_distances = quantities.find('d') != std::string::npos;
        const bool want_vectors = quantities.find('D') != std::string::npos;
        const bool through_autograd = differentiate && (want_distances || want_vectors);

        VesinOptions options;
        std::memset(&options, 0, sizeof(options));
        options.cutoff = cutoff_;
        options.full = full_list_;
        options.sorted = sorted_;
        options.algorithm = parse_algorithm(algorithm_);
        options.n_threads = static_cast<int32_t>(n_threads_ == 0 ? at::get_num_threads() : n_threads_);
        options.return_shifts = quantities.find('S') != std::string::npos || (through_autograd && box.requires_grad());
        // the gradient needs both the distances and the vectors
        options.return_distances = want_distances || through_autograd;
        options.return_vectors = want_vectors || through_autograd;
        options.skin = 0.0;

        if (list_.device.type != VesinUnknownDevice && list_.device.type != device.type) {
            vesin_free(&list_);
            from_torch_allocator_ = false;
        }
        if (!from_torch_allocator_ && device.type == VesinCUDA) {
            const char* error_message = nullptr;
            const auto status = vesin_hip_set_output_allocator(
                &list_, device, vesin_amd_torch_allocate, vesin_amd_torch_release, nullptr, &error_message
            );
            if (status != EXIT_SUCCESS) {
                throw std::runtime_error(std::string("failed to compute neighbors: ") + error_message);
            }
            from_torch_allocator_ = true;
        }

        auto points_data = points.detach().contiguous();
        auto box_data = box.detach().contiguous();
        const char* error_message = nullptr;
        const auto status = vesin_hip_neighbors_on_stream(
            reinterpret_cast<const double (*)[3]>(points_data.data_ptr<double>()),
            static_cast<size_t>(points_data.size(0)),
            reinterpret_cast<const double (*)[3]>(box_data.data_ptr<double>()),
            periodic.data_ptr<bool>(),
            device,
            options,
            &list_,
            points.is_cuda() ? PairGeometry::current_stream(points.device()) : nullptr,
            &error_message
        );
        if (status != EXIT_SUCCESS) {
            throw std::runtime_error(std::string("failed to compute neighbors: ") + error_message);
        }

        static_assert(sizeof(size_t) == sizeof(int64_t), "pairs are handed out as 64-bit integers");
        const auto length = static_cast<int64_t>(list_.length);
        const auto on_device = torch::TensorOptions().device(points.device());
        // what the backward step will read must outlive the next calculation on this list: never a view then
        const bool own_copy = copy || through_autograd;
        // Instead of a copy the tensors take the arrays over, unless those are much larger than their rows (a list
        // that saw a large system keeps large arrays: a caller who collects the lists of many small systems would
        // hold all that room).
        void* const arrays[4] = {list_.pairs, list_.shifts, list_.distances, list_.vectors};
        bool hand_over = false;
        if (own_copy && from_torch_allocator_ && length > 0 &&
            static_cast<size_t>(length) >= vesin_hip_output_capacity(&list_) / 2) {
            const char* detach_message = nullptr;
            hand_over = vesin_hip_detach_outputs(&list_, nullptr, &detach_message) == EXIT_SUCCESS;
        }
        const auto wrap = [&](void* data, std::vector<int64_t> shape, torch::ScalarType dtype) {
            if (length == 0 || data == nullptr) {
                return torch::empty(shape, on_device.dtype(dtype));
            }
            if (hand_over) {
                return adopt_array(data, shape, dtype, points.device());
            }
            auto view = torch::from_blob(data, shape, on_device.dtype(dtype));
            return own_copy ? view.clone() : view;
        };

        auto pairs = wrap(arrays[0], {length, 2}, torch::kInt64);
        auto shifts = torch::Tensor();
        if (options.return_shifts) {
            shifts = wrap(arrays[1], {length, 3}, torch::kInt32);
        }
        auto distances = torch::Tensor();
        if (options.return_distances) {
            distances = wrap(arrays[2], {length}, torch::kFloat64);
        }
        auto vectors = torch::Tensor();
        if (options.return_vectors) {
            vectors = wrap(arrays[3], {length, 3}, torch::kFloat64);
        }
        if (hand_over) {
            // (an array that no tensor took: there is none today, every array the list holds was asked for)
            const bool taken[4] = {true, shifts.defined(), distances.defined(), vectors.defined()};
            for (int k = 0; k < 4; k++) {
                if (arrays[k] != nullptr && !taken[k]) {
                    vesin_amd_torch_release(arrays[k], nullptr);
                }
            }
        }

        if (through_autograd) {
            auto shifts_or_nothing = shifts.defined() ? shifts : torch::empty({0, 3}, on_device.dtype(torch::kInt32));
            auto outputs = PairGeometry::apply(points, box, pairs, shifts_or_nothing, distances, vectors, any_periodic);
            distances = outputs[0];
            vectors = outputs[1];
        }

        auto output = std::vector<torch::Tensor>();
        output.reserve(quantities.size());
        for (const char letter : quantities) {
            switch (letter) {
            case 'i':
                output.push_back(pairs.select(1, 0));
                break;
            case 'j':
                output.push_back(pairs.select(1, 1));
                break;
            case 'P':
                output.push_back(pairs);
                break;
            case 'S':
                output.push_back(shifts);
                break;
            case 'd':
                output.push_back(distances);
                break;
            default:
                output.push_back(vectors);
                break;
            }
        }
        return output;
    }

    double cutoff() const { return cutoff_; }
    bool full_list() const { return full_list_; }
    bool sorted() const { return sorted_; }
    const std::string& algorithm() const { return algorithm_; }
    int64_t n_threads() const { return n_threads_; }

private:
    double cutoff_;
    bool full_list_;
    bool sorted_;
    std::string algorithm_;
    int64_t n_threads_;
    VesinNeighborList list_ = VesinNeighborList();
    bool from_torch_allocator_ = false; // the arrays of list_ come from PyTorch's caching allocator
};

} // namespace vesin_amd_torch

TORCH_LIBRARY(vesin_amd, m) {
    m.def("adopt(int pointer, int[] shape, ScalarType dtype, int device) -> Tensor", &vesin_amd_torch::adopt);
}

TORCH_LIBRARY(vesin, m) {
    using vesin_amd_torch::NeighborListHolder;
    const std::string no_doc;

    m.class_<NeighborListHolder>("_NeighborList")
        .def(
            torch::init<double, bool, bool, std::string, int64_t>(),
            no_doc,
            {torch::arg("cutoff"),
             torch::arg("full_list"),
             torch::arg("sorted") = false,
             torch::arg("algorithm") = "auto",
             torch::arg("n_threads") = 0}
        )
        .def(
            "compute",
            &NeighborListHolder::compute,
            no_doc,
            {torch::arg("points"),
             torch::arg("box"),
             torch::arg("periodic"),
             torch::arg("quantities"),
             torch::arg("copy") = true}
        )
        .def_pickle(
            [](const c10::intrusive_ptr<NeighborListHolder>& self) {
                // a dictionary of mixed values can only be made untyped first
                c10::impl::GenericDict state(c10::StringType::get(), c10::AnyType::get());
                state.insert("cutoff", self->cutoff());
                state.insert("full_list", self->full_list());
                state.insert("sorted", self->sorted());
                state.insert("algorithm", self->algorithm());
                state.insert("n_threads", self->n_threads());
                return c10::impl::toTypedDict<std::string, c10::IValue>(state);
            },
            [](c10::Dict<std::string, c10::IValue> state) {
                return c10::make_intrusive<NeighborListHolder>(
                    state.at("cutoff").toDouble(),
                    state.at("full_list").toBool(),
                    state.at("sorted").toBool(),
                    state.at("algorithm").toStringRef(),
                    state.at("n_threads").toInt()
                );
            }
        );
}
