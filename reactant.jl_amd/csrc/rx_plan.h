// Fusion planning: rx::Graph -> fusion groups -> one HIP translation unit plus a
// launch list.  The runtime compiles the text with hiprtc and replays the list.
#pragma once
#include "rx_ir.h"

namespace rx {

struct BufferDesc {
  // Fault: the device's fault word, a 32-bit word in pinned host memory that a kernel sets when a bounded wait for
  // another workgroup expires; the runtime checks it wherever the host waits for the device
  enum Kind { Param, Const, Temp, Scratch, Fault } kind = Temp;
  TType ty;                    // element type / shape (Scratch: bytes only)
  int64_t bytes = 0;
  int param_index = -1;        // Param
  std::vector<uint8_t> data;   // Const: storage bytes uploaded once at compile time
  int first_def = -1;          // index of the launch that writes it (Temp/Scratch)
  int last_use = -1;           // index of the last launch that touches it
  bool is_result = false;
};

struct Launch {
  std::string kernel;          // symbol in the translation unit
  std::string kind;            // "map" | "reduce" | "reduce_final" | "row" | "dot" | "gemm_*"
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {1, 1, 1};
  unsigned lds_bytes = 0;
  std::vector<int> args;       // buffer ids, in kernel parameter order
  int n_outputs = 1;           // trailing args written by the kernel
  double algo_bytes = 0;       // compulsory HBM traffic: distinct inputs once + outputs once
  double flops = 0;            // contraction flops (2*M*N*K) for dot groups
  std::string desc;            // human-readable summary of the fused ops
};

struct Plan {
  std::string source;                  // HIP text for all kernels of the module
  std::vector<BufferDesc> buffers;
  std::vector<Launch> launches;
  std::vector<int> result_buffers;     // per @main result: buffer id
  std::vector<TType> param_types, result_types;
  std::vector<int> aliasing_output;    // per argument: result index it may alias, or -1
  // Counts over the live nodes of the module as written (what XLA's HloCostAnalysis reports for a module, reference
  // deps/ReactantExtra/API.cpp:3224-3260): arithmetic operations (2 M N K per product, one per element of every other
  // arithmetic op and of every reduced element), elements of transcendental ops, and per-op bytes read and written
  double hlo_flops = 0, hlo_transcendentals = 0, hlo_bytes_accessed = 0, hlo_output_bytes = 0;
  double hlo_operand_bytes[2] = {0, 0};
  std::string report() const;          // text summary for debugging
};

struct PlanOptions {
  bool xcd_slabs = true;        // XCD-aware tile order for kernels with shifted loads
  int64_t slab_min_numel = 1 << 22;  // smallest output that uses it
  int64_t slab_order_min_numel = 1 << 22;  // smallest plain map with loads shifted along the slowest dimension that takes the XCD slab order
  bool mfma = true;             // use the MFMA GEMM skeletons for eligible dot_generals
  bool dot_as_reduce = true;    // dot_generals with a vector-like operand run as multiply + reduce
  bool fuse_dot_operands = true;  // a dot operand that expands much smaller data is evaluated inside the GEMM's tile loads
  bool split_k = true;          // matrix products with few output tiles and a long contraction: K in slices, partial products, a reduction
  bool chain_convs = true;      // two 16-bit convolutions with only channel-wise elementwise ops and padding between them share the padded grid: no map in between
  bool product_epilogues = true;  // the elementwise ops that consume a product or convolution run in its kernel (off: a map after it; for comparisons)
  int conv_tails = 1;           // the elementwise chain after a convolution is written where a window, reduction or layout change reads it, so that it runs in the convolution's kernel: 1 when it ends in a type narrower than the f32 accumulators, 2 always, 0 never
  bool nhwc_pools = true;       // pooling windows (and the elementwise ops and padding around them) between two 16-bit convolutions run on the channel-minor layout: no transposes
  bool merge_parameter_maps = true;  // plain maps that read only the module's arguments run first, several of them as one launch
  bool nhwc_regions = true;     // the same for regions with several readers per value (residual additions): transposed once on the way in and out where needed
  double nhwc_region_ratio = 1.5;   // a region is rebuilt when the transposes that disappear move this many times the bytes of those that are added (two residual blocks: 3 against 2 tensors, 0.129 -> 0.115 ms)
  bool pad_into_pools = true;   // zero padding of a pooled value (windows that do not overlap) moves onto the pooling's operand: no padding map
  bool epilogue_init = true;    // a bias added to a product on the streaming skeletons becomes the accumulators' first values
  bool row_fusion = true;       // fuse row reductions with their elementwise consumers
  bool lds_stencil = true;      // 3-D maps that read an input at several offsets stage it through LDS halo tiles
  int slab_ytiles = 0;          // stencil kernels: y-tiles per XCD slab (0: one slab per XCD)
  int lds_tile[3] = {3, 4, 128};  // outputs per workgroup tile (slowest .. fastest dimension)
  // full reductions in one launch: every workgroup publishes its partial as flagged words and the
  // workgroup with the last index waits for all of them and combines.  Off: it saves the 1-workgroup
  // combine launch (1.4 us of an 85 us step over 2^26 elements, 1.2 us of a 485 us FP8 step), and it
  // adds a wait between workgroups whose expiry would go unreported.  (An earlier form with a
  // device-scope release fence before a ticket -- an L2 write-back on this multi-die part -- was 2x slower.)
  bool single_pass_reduce = false;
  bool single_pass_scan = true;      // long scanned rows in one launch (chunk totals travel as flagged words)
  bool window_reduce_vectors = true;  // reductions over 16-bit elements that keep the minor dimension (pooling windows): eight outputs per thread
  bool reduce_row_blocks = true;   // reductions whose kept minor dimension is one vector long (skinny matrix products): a thread takes four values of the next kept dimension too
  bool lds_transpose = true;       // maps with transposed reads: stage 64x64 tiles through LDS
  bool branchless_guards = true;   // stencil kernels: evaluate pad/update guards as selects when every guarded read is a tile read
  bool clamp_pad_reads = true;     // maps over 8- and 16-bit elements: padded reads at clamped positions and a select, so that a lane's loads combine
  bool stencil_fuse_steps = true;  // two consecutive stencil steps in one kernel: the first step's result lives only in LDS
  int lds_tile2[3] = {4, 8, 64};   // outputs per workgroup tile of the two-step kernel
  int lds2_threads = 512;          // its workgroup size
  bool stencil_march2 = true;      // two-step kernel marching along the slowest dimension instead of 3-D tiles
  int march2_tile[2] = {8, 64};    // its outputs per plane (rows, columns)
  bool march2_edge = true;         // a nearly empty last tile column is covered by tiles a quarter as wide, four times as tall
  int march2_planes = 22;          // planes per workgroup, about (the extent is cut into equal chunks)
  bool transpose_vectors = true;   // transposing maps move 16-byte vectors where the dimensions allow it
  bool transpose_offsets = true;   // a transposed read of a padded or sliced operand is staged through the LDS tiles too
  int transpose_block = 8;         // their tiles are taken in blocks of this many by this many (1: plain order)
  int march2_lds_ballast = 0;   // bytes of LDS the marching stencil kernel declares and never uses: lowers its occupancy (measurements only)
  int march2_prefetch = 2;   // planes that the marching stencil kernel requests ahead of their use (1 or 2)
  // Runs of in-place update steps over small arrays (time loops of stencils): up to `chain_steps`
  // consecutive steps per launch, the arrays held in LDS tiles in between (0: 64 for vectors, 16
  // otherwise; 1: off)
  int chain_steps = 0;
  int chain_tile[3] = {0, 0, 0};     // outputs per workgroup (slowest .. fastest dimension of the array's rank; zeros: default per rank)
  int64_t chain_lds_bytes = 64 * 1024;  // LDS a workgroup may use for the tiles
  int64_t chain_rank3_numel = 1 << 18;  // rank-3 steps up to this many elements are chained all the same (four per launch)
  int chain_max_rank = 2;            // rank-3 steps are bound by index arithmetic in such a kernel, not by launches: left as maps
  bool chain_fixed_cells = true;     // a thread keeps the same box cells (and their coordinates in registers) through all steps
  int chain_threads = 0;             // workgroup size (0: by the number of staged cells)
  double chain_redundancy = 4.1;     // largest ratio of staged cells (tile plus halo) to tile cells
  bool in_place_updates = true;   // dynamic_update_slice over a temporary nobody reads later writes only its box, into the operand's buffer
  bool shifted_vector_loads = true;  // loads at constant offsets become aligned vector loads of neighbouring vectors
  bool excess_precision = true; // narrow-float arithmetic stays in f32 inside a kernel (rounded at stores and converts)
  bool nt_loads = true;         // non-temporal hint on inputs that are read exactly once
  bool nt_stores = true;        // non-temporal hint on map outputs
};

Plan make_plan(const Graph& g, const PlanOptions& opt);

}  // namespace rx
