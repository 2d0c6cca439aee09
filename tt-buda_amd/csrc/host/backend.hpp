// Host side of the tensor boundary: the descriptor types and the tt::backend free functions that
// pybuda binds (pybuda/csrc/backend_api/backend_api.cpp:409-591, 622-625, 688-723), implemented on
// queues that live in MI355X HBM.  All GPU work goes through the C ABI of include/ttbfp.h.
#pragma once

#include <array>
#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "data_format.hpp"

namespace tt {

// backend_api.cpp:622-625
enum class DEVICE_STATUS_CODE : int { Success = 0, RuntimeError = 1, TimeoutError = 2 };
// backend_api.cpp:321-329
enum class IO_TYPE : int { Queue = 0, RandomAccess = 1, Invalid = 0xff };
enum class IO_LAYOUT : int { Tilized = 0, Flat = 1, Invalid = 0xff };
// The only device kind this backend drives.
enum class DEVICE : int { Hip = 0, Invalid = 0xff };
// The part it drives, and how a backend object is used (the reference's BackendDevice and DeviceMode arguments of
// BackendConfig, pybuda/csrc/backend_api/backend_api.cpp:243-260); kept so that the constructor takes the same arguments.
enum class ARCH : int { MI355X = 0, Invalid = 0xff };
enum class DEVICE_MODE : int { CompileAndRun = 0, CompileOnly = 1, RunOnly = 2 };

// pybuda/csrc/tt_torch_device/tt_device.hpp:205-210
template <typename T>
inline T align_up_tile(T d)
{
    return static_cast<T>((d + 31) / 32 * 32);
}

// tt_backend_config as far as this backend reads it (backend_api.cpp:243-281).  ignore_data_format_precision is the
// golden-precision switch: false (the default of a device backend) keeps every queue in its declared DataFormat, so
// tensors are quantized on the way in and the matmul runs on the dequantized values; true ("run backend at full precision",
// what the reference's Golden device does unless told otherwise, backend_api.cpp:268-270, pybuda/pybuda/verify/config.py:67)
// keeps queues unquantized and evaluates in fp32.
struct tt_backend_config {
    DEVICE type = DEVICE::Hip;
    ARCH arch = ARCH::MI355X;
    DEVICE_MODE mode = DEVICE_MODE::CompileAndRun;
    int optimization_level = 0;
    std::string output_dir;
    std::string soc_descriptor_path;
    std::string cluster_descriptor_path;
    bool ignore_data_format_precision = false;
    std::string perf_desc_args;
    std::string runtime_args;
};

// backend_api.cpp:384-407
struct Stride {
    std::vector<std::pair<int, int>> xy_offsets;
    int stride = -1;
};

// Row-major view of a tensor, at most 4-D: shape (w, z, r, c), strides in BYTES, outermost first
// (backend_api.cpp:489-560; pybuda/csrc/lower_to_buda/common.hpp:251-258).  `owner` keeps whatever
// object backs `ptr` alive (a Python tensor when built from one).
struct tt_PytorchTensorDesc {
    const void *ptr = nullptr;
    std::uint32_t itemsize = 0;
    DataFormat format = DataFormat::Invalid;
    std::array<std::uint32_t, 4> shape = {1, 1, 1, 1};
    std::array<std::uint32_t, 4> strides = {0, 0, 0, 0};
    std::uint32_t dim = 4;
    std::shared_ptr<void> owner;

    tt_PytorchTensorDesc() = default;
    tt_PytorchTensorDesc(const void *p, std::uint32_t isz, DataFormat f, std::array<std::uint32_t, 4> sh,
                         std::array<std::uint32_t, 4> st, std::uint32_t d = 4, std::shared_ptr<void> own = nullptr)
        : ptr(p), itemsize(isz), format(f), shape(sh), strides(st), dim(d), owner(std::move(own))
    {
    }
    std::uint64_t elements() const { return (std::uint64_t)shape[0] * shape[1] * shape[2] * shape[3]; }
};

// Result of tilize_tensor: `num_buffers` buffers (one per queue grid core) of `buf_size_bytes`
// each, back to back at `ptr` (backend_api.cpp:562-591).
struct tt_TilizedTensorDesc {
    const void *ptr = nullptr;
    std::uint32_t num_buffers = 0;
    std::uint32_t buf_size_bytes = 0;
    DataFormat format = DataFormat::Invalid;

    tt_TilizedTensorDesc() = default;
    tt_TilizedTensorDesc(const void *p, std::uint32_t n, std::uint32_t b, DataFormat f)
        : ptr(p), num_buffers(n), buf_size_bytes(b), format(f)
    {
    }
};

// Geometry of a device queue (backend_api.cpp:409-487).  One entry holds `t` slices of
// (grid_r * mblock_m * ublock_rt) x (grid_c * mblock_n * ublock_ct) tiles.
struct tt_dram_io_desc {
    std::string netlist_path;
    std::string queue_name;
    std::uint32_t bufq_grid_dim_r = 1, bufq_grid_dim_c = 1;
    std::uint32_t bufq_num_slots = 1;
    std::uint32_t ublock_rt = 1, ublock_ct = 1;
    std::uint32_t mblock_m = 1, mblock_n = 1;
    std::uint32_t tile_height = 32, tile_width = 32;
    std::uint32_t t = 1;
    std::uint32_t input_count = 1;
    std::uint32_t hstack_factor = 1, vstack_factor = 1, stack_row_major = 1;
    DataFormat bufq_target_format = DataFormat::Invalid;
    std::vector<std::pair<std::uint32_t, std::uint16_t>> bufq_start_addr_channel;
    std::uint32_t bufq_entry_size = 0;
    IO_TYPE io_type = IO_TYPE::Queue;
    Stride s_descriptor;
    DEVICE backend_type = DEVICE::Hip;
    IO_LAYOUT layout = IO_LAYOUT::Tilized;
    // Two properties the reference's backend reads from the netlist the descriptor names rather than
    // from the descriptor: the order of micro blocks inside a macro block (the queue line's
    // "ublock_order: r|c", pybuda/csrc/lower_to_buda/queue.cpp:24-28; 0 = r, 1 = c) and whether every
    // tile carries its header and padding (pybuda/csrc/balancer/balancer_utils.hpp:24-27).
    std::uint32_t ublock_order = 0;
    std::uint32_t tile_header = 0;

    std::uint32_t rows() const { return bufq_grid_dim_r * mblock_m * ublock_rt * tile_height; }
    std::uint32_t cols() const { return bufq_grid_dim_c * mblock_n * ublock_ct * tile_width; }
};

// Rounding of step 7 of the Float->BFP conversion (docs/public/dataformats.rst:81).  Read once
// from the environment variable TTBFP_ROUNDING ("truncate", the default, or "nearest").
int conversion_rounding();

// The object pybuda calls BackendApi (backend_api.cpp:666-674).  The reference builds its queues
// from a netlist; here they are declared one by one with create_queue.
class tt_backend {
   public:
    static std::shared_ptr<tt_backend> create(int device = 0, const tt_backend_config &config = tt_backend_config());
    ~tt_backend();

    DEVICE_STATUS_CODE initialize();
    DEVICE_STATUS_CODE finish();
    DEVICE_STATUS_CODE wait_for_idle();

    // Allocates `num_slots` entries of HBM for a queue and registers it under `name`.  The entry is cut
    // over grid_r x grid_c buffers; inside a buffer the tiles follow the order of TileLayout::map
    // (pybuda/csrc/balancer/types.cpp:629-648).  Buffer b keeps its num_slots entries together, the
    // buffers follow one another in HBM.
    tt_dram_io_desc create_queue(const std::string &name, DataFormat format, std::uint32_t t, std::uint32_t mblock_m,
                                 std::uint32_t mblock_n, std::uint32_t ublock_rt = 1, std::uint32_t ublock_ct = 1,
                                 std::uint32_t num_slots = 2, IO_TYPE io_type = IO_TYPE::Queue,
                                 std::uint32_t input_count = 1, std::uint32_t grid_r = 1, std::uint32_t grid_c = 1,
                                 std::uint32_t ublock_order = 0, bool tile_header = false);
    tt_dram_io_desc get_queue_descriptor(const std::string &name) const;
    // The format of the tiles a queue holds in HBM: its declared format, or with ignore_data_format_precision the
    // full-precision stand-in (Float32 for the formats with an 8-bit exponent, Float16 for those with five).
    DataFormat queue_storage_format(const std::string &name) const;
    // The largest number of push_input / get_output / run_matmul conversions that ever ran on this queue at one time.
    std::uint32_t queue_max_in_flight(const std::string &name) const;
    // conversions (pushes and reads) of the queue that hold a reservation or a pin right now
    std::uint32_t queue_in_flight(const std::string &name) const;
    const tt_backend_config &config() const { return config_; }

    // out = epilogue(in0 * weight + bias): the matmul op of a netlist program, evaluated with the
    // Bfp8_b-weight GEMM.  in0 and out are Float16_b queues, weight a Bfp8_b RandomAccess queue
    // holding W[K,N], bias (optional, "" = none) a Float16_b RandomAccess queue whose row 0 is
    // broadcast (pybuda/pybuda/op/eval/buda/matmul.py:233-249).  With ignore_data_format_precision the queues hold
    // unquantized fp32 tiles whatever their declared formats, and the product is an fp32 matmul on them.  Consumes one entry of in0 and
    // produces one entry of out.  gelu: apply GELU to the result, in the form `approximate` names ("none": erf form,
    // "tanh": pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:42-49; anything else is an error as it is there).
    DEVICE_STATUS_CODE run_matmul(const std::string &in0, const std::string &weight, const std::string &bias,
                                  const std::string &out, bool gelu, int timeout_s = 10, const std::string &approximate = "none");

    const std::string &id() const { return id_; }

   private:
    tt_backend(int device, const tt_backend_config &config);
    int device_;
    tt_backend_config config_;
    std::string id_;
    std::vector<std::string> queues_;
};

namespace backend {

// Rows and columns of the tensor that are not multiples of 32 are padded to the entry's tiles inside the pack launch
// (zeros; with tile_broadcast_r / tile_broadcast_c a dimension of one is copied through its tile instead, the "replicate"
// mode of pad_pytorch_tensor_to_buda, pybuda/pybuda/tensor.py:848-856).  timeout_in_seconds bounds the wait for free slots.
DEVICE_STATUS_CODE push_input(const tt_dram_io_desc &q, const tt_PytorchTensorDesc &tensor, const bool push_one,
                              const int timeout_in_seconds, const int ram_ptr, const bool tile_broadcast_r = false,
                              const bool tile_broadcast_c = false);
DEVICE_STATUS_CODE push_input(const tt_dram_io_desc &q, const tt_TilizedTensorDesc &tensor, const int timeout_in_seconds,
                              const int ram_ptr);
// narrow_r / narrow_c (0: the whole entry): the result keeps only that many rows / columns of every slice
// (narrow_buda_tensor_to_pytorch, pybuda/pybuda/tensor.py:879-954, inside the unpack launch).
DEVICE_STATUS_CODE get_output(const tt_dram_io_desc &q, tt_PytorchTensorDesc &out, const bool pop_one,
                              const int timeout_in_seconds, const int rd_ptr, const std::uint32_t narrow_r = 0,
                              const std::uint32_t narrow_c = 0);
DEVICE_STATUS_CODE pop_output(const tt_dram_io_desc &q, const bool pop_one, const int timeout_in_seconds);
DEVICE_STATUS_CODE translate_addresses(tt_dram_io_desc &q);

template <typename T>
DEVICE_STATUS_CODE free_tensor(T &desc);

// Row-major host (or device) tensor -> tiles in the queue's format, in backend-owned pinned host
// memory; release with free_tensor.  Throws std::runtime_error on failure, as the reference does.
tt_TilizedTensorDesc tilize_tensor(const tt_dram_io_desc &q, const tt_PytorchTensorDesc &tensor);

// Host tensor of up to four dimensions -> 4-D, rows and columns zero-padded to whole tiles, contiguous, in backend-owned
// pinned memory (pybuda/csrc/tt_torch_device/tt_device.cpp:153-189).  Throws std::runtime_error on failure.
tt_PytorchTensorDesc pad_to_buda_shape(const tt_PytorchTensorDesc &tensor);

// Device and pinned-host blocks the pools behind push_input / get_output / tilize_tensor / run_matmul have allocated so far:
// constant in steady state.
std::uint64_t pool_allocations();

template <typename T>
void binarize_tensor(const T &desc, std::string file_path);
template <typename T>
void debinarize_tensor(T &desc, std::string file_path);

// Bytes one queue needs in device memory (backend_api.cpp:710-722): a 32-byte queue header, then per
// entry either tiles with their 32-byte header (balancer_utils.hpp:24-27) or, untilized, the bare
// row-major elements.
std::uint32_t get_io_size_in_bytes(DataFormat df, bool is_untilized, std::uint32_t ublock_ct, std::uint32_t ublock_rt,
                                   std::uint32_t mblock_m, std::uint32_t mblock_n, std::uint32_t t, std::uint32_t entries,
                                   std::uint32_t tile_height = 32, std::uint32_t tile_width = 32);

// Text of the last failure reported by a status code on this thread.
std::string last_error();

}  // namespace backend
}  // namespace tt
