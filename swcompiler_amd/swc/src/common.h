// Shared vocabulary of the SWC API: data types, layouts, devices and the
// Config record that selects a backend.  Names and enumerators are the
// reference's (src/common.h:17-180) because user programs spell them; the
// fields below the "HIP target" comment are additive.
#ifndef SWC_COMMON_H_
#define SWC_COMMON_H_

#include <algorithm>
#include <climits>
#include <cstddef>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

enum class DataType { Float_t, Double_t, Int8_t, Int32_t };

enum ParallelStrategy { SLICE, TILING, MEM_SAVING, COMM_SAVING };
enum BytesProto { ONE_BYTE_AS_INT, FOUR_BYTES_AS_FLOAT };
enum NetTopology { FC_MESH_NET, STAR_NET, RING_NET, TREE_NET };

// Settings of a training program (Config::train_mode; reference: src/common.h:40-58).  snapshot: every that many
// iterations the parameters, momenta and the iteration count are written to snapshot_iter<N>.model (0: never).
struct TrainingConfig {
    std::string optimizer;
    float lr{0.001f};
    float decay{0.001f};
    float momentum{0.9f};
    size_t batch{1};
    size_t snapshot{0};
    size_t max_epoch{1};
    size_t max_iters{0};
    size_t display{0};
    BytesProto label_bytes{ONE_BYTE_AS_INT};
    BytesProto data_bytes{FOUR_BYTES_AS_FLOAT};
    std::string train_data_file;
    size_t train_data_samples{0};
};

struct Config {
    bool train_mode{false};     // Engine::compile adds gradient ops and optimizer updates; the program loops over train_config's records
    // targets of the reference that this build does not have: setting one makes Engine::compile / Codegen stop with a message
    bool mkldnn{false};
    bool cuda{false};
    bool cublas{false};
    bool cuda_stream{false};
    bool mpi{false};
    int mpi_size{1};
    TrainingConfig train_config;
    // inference over a file of records: `while (loader.next(label, data))` around the op sequence
    bool use_dataloader{false};
    std::string dataloader_src;                  // the record file
    BytesProto label_bytes{ONE_BYTE_AS_INT};     // how a record stores its label ...
    BytesProto data_bytes{FOUR_BYTES_AS_FLOAT};  // ... and its data elements
    size_t dataloader_samples{0};                // records in the file
    size_t display{0};                           // > 0: the display tensors are printed every that many iterations
    bool enable_lowering{true};                  // LoweringPass rewrites FC ops into MatrixMatrixMul + bias add (false: left whole)
    bool benchmark{false};                       // training programs: no snapshots, no display output
    // settings of the reference's multi-rank generators: carried for source compatibility, read by nothing here
    ParallelStrategy parallel_preference{MEM_SAVING};
    bool force_data_parallel{false};
    bool handcraft_parallel{false};
    bool geneticalgo_opt_parallel{false};
    bool compute_op_annotation{false};
    bool comm_op_annotation{false};
    NetTopology net_topo{FC_MESH_NET};
    bool decentralized_optimizer{false};

    // ---- HIP target (MI355X / gfx950) ----
    bool hip{false};            // compile the graph for libswc_hip on one GPU
    int hip_device{0};          // device ordinal passed to swc_hip_init
    bool hip_fusion{true};      // fold bias/BN/ReLU into GEMM/conv epilogues, BN+ReLU(+pool) into one pass
    size_t time_iters{0};       // > 0: generated program repeats the op sequence and prints ms/iteration
    bool hip_prefetch{false};   // with use_dataloader and hip_graph: the next batch is read and uploaded (second stream) while this one is computed
    bool hip_graph{false};      // with time_iters or use_dataloader: record the device ops of an iteration into one HIP graph and replay that
    bool dump_outputs{false};   // generated program writes every graph output to <name>.bin (raw fp32/int32)
};

enum OpType { TENSOR_OP, BASIC_OP, DL_OP };
enum NodeType { TENSOR_NODE, OP_NODE };
enum TensorType { D5 = 5, D4 = 4, D3 = 3, D2 = 2, D1 = 1, D0 = 0, UNKNOWN = -1 };

typedef enum { layout_default = 0, layout_nchw, layout_nhwc, layout_nc, layout_cn } mem_layout_t;

enum class TensorInitType { NONE, CONSTANT, ZERO, XAVIER, FILE, PARENTOP };
enum class DeviceType : int { CPU, GPU };
enum class PrintStreamType { COUT, FILE };

struct Device {
    int rank{0};
    DeviceType type{DeviceType::CPU};
    int id{0};
    Device(int r = 0, DeviceType t = DeviceType::CPU, int i = 0) : rank(r), type(t), id(i) {}
    friend bool operator==(const Device &a, const Device &b) {
        return a.rank == b.rank && a.type == b.type && a.id == b.id;
    }
    friend bool operator!=(const Device &a, const Device &b) { return !(a == b); }
};

namespace std {
template <> struct hash<Device> {
    size_t operator()(const Device &d) const {
        return (size_t)d.rank * 1000003u ^ ((size_t)d.type << 16) ^ (size_t)d.id;
    }
};
} // namespace std

#define NCHW2NHWC {0, 2, 3, 1}
#define NHWC2NCHW {0, 3, 1, 2}

// Removes the first element equal to `victim`; returns whether one was found.
template <typename U, typename V> int delVecMember(std::vector<U> &vec, V &victim) {
    auto it = std::find(vec.begin(), vec.end(), victim);
    if (it == vec.end()) return 0;
    vec.erase(it);
    return 1;
}

#endif
