// The problem sizes at which an operation changes kernels, in one place, each
// with the measurement that set it (MI355X, one GPU; whole calls timed on the
// device unless it says otherwise). The kernels' own capacity limits (what a
// layout can hold) stay with the kernels; what is here decides between two
// kernels that could both serve the shape.
#ifndef MOPS_AMD_DISPATCH_THRESHOLDS_HPP
#define MOPS_AMD_DISPATCH_THRESHOLDS_HPP

#include <cstddef>
#include <cstdint>

namespace mops::amd::thresholds {

// ---- HPE (hpe.hip) ---------------------------------------------------------
/// Rows from which the vjp goes by feature (the table turned round by a launch
/// in front, accumulators in registers) instead of a workgroup per few rows
/// with accumulators in LDS, which with thousands of rows is bound by its LDS
/// add instructions. At 1000 rows by feature is the slower way (the extra
/// launch). 8192 rows, 2000 monomials of order 4: 169 -> 64 us.
constexpr int32_t HPE_VJP_BY_FEATURE_ROWS = 4096;
/// Rows from which the forward pass has a lane per row (a workgroup per 64 or
/// 128 rows): fewer workgroups than about one per compute unit leave the
/// kernel with a workgroup per few rows ahead (8192 rows: 24 us against 35).
constexpr int32_t HPE_FORWARD_LANE_PER_ROW_ROWS = 200 * 64;

// ---- SAP (sap_mfma.hip) ----------------------------------------------------
/// Tiles of 16 rows per wavefront of the device from which a launch has as many
/// workgroups as the device holds, each building the dense table once and
/// walking over tiles, instead of a workgroup (and a table build) per 128 rows.
/// nA, nB, nO = 13, 7, 20 over 65 000 to 560 000 rows: the forward pass gains
/// from one tile per wavefront on (200 000 rows, f32: 33.3 -> 30.0 us; f64 at
/// 100 000: 30.0 -> 25.9), the vjp from two (400 000 rows, f32: 88.9 -> 83.5
/// us; with one, 140 000 rows take 41.4 instead of 35.9 us).
constexpr int64_t SAP_FORWARD_WALK_TILES_PER_WAVE = 1;
constexpr int64_t SAP_VJP_WALK_TILES_PER_WAVE = 2;

// ---- OPSA / OPSAW (opsa.hip) -----------------------------------------------
/// Forward pass: segments are cut every so many positions of the sorted index,
/// and the pieces added by a second launch, when the average segment is twice
/// as long (pooling over whole structures: one wavefront per segment would
/// leave the device idle). 50 rows of 2400 edges: 94 -> 21 us in f32.
constexpr int OPSA_SPLIT_POSITIONS = 256;
/// vjp: columns of A up to which the per-edge kernel keeps a receiver's rows
/// of grad_output as matrix operands in registers (one to four tiles of 16);
/// beyond, the LDS-staged kernels. 60 000 edges, K = L = 48: 34 us against 82
/// (f32), 61 against 150 (f64); K = L = 64: 58 against 140, 107 against 552;
/// K = 56, L = 128: 118 against 507, 177 against 994; OPSAW K = L = 64: 97
/// against 220, 133 against 566.
constexpr int32_t OPSA_VJP_ROWS_IN_REGISTERS = 64;

// ---- the edges of every sender (grad_W of OPSAW and SASAW) -------------------
/// Index reads (edges x workgroups) up to which every workgroup finds its
/// senders' edges by reading the whole sender index; beyond, a counting sort
/// of the edges by sender (at 60 000 edges the sort costs more than the reads:
/// 52 us against 32 for the whole OPSAW vjp).
constexpr size_t SENDER_SCAN_LIMIT = 100u * 1000 * 1000;
/// Edges per sender on average up to which the lists are kept in slots (the
/// index in 4 parts, 32 places per sender and part: a part then holds 12 edges
/// of a sender on average; a sender that overflows is served by a wavefront
/// reading the whole index). OPSAW, 60 000 edges over 2000 senders, L = 32,
/// f32: 33 -> 22 us for the whole vjp.
constexpr int32_t SLOT_MEAN_EDGES = 48;
/// Edges per sender on average up to which SASAW lists by arrival (128 places
/// per sender): 1000 nodes x 60 edges, whole vjp 87.6 -> 76.6 us (f32), 143.8
/// -> 115.3 (f64) against the kernels of sasaw_mfma.hip; at 100 per sender the
/// lists overflow (375 against 101 us).
constexpr int32_t ARRIVAL_MEAN_EDGES = 64;
/// Nodes from which the lists are made by arrival (one look at every edge, an
/// integer atomic each) rather than in slots (edges x nodes / 16 tests).
/// SASAW f32 vjp at 30 edges per node, by arrival / in slots: 2000 nodes 66.7 /
/// 60.7 us, 3000: 93.8 / 92.8, 4000: 113.7 / 114.0, 6000: 170 / 179, 8000: 233
/// / 255, 20 000: 682 / 820. OPSAW f32 vjp: 2000 senders 27.6 / 22.6, 3000:
/// 33.4 / 29.6, 4000: 37.6 / 39.3, 6000: 48 / 75, 20 000: 156 / 212.
constexpr int32_t ARRIVAL_NODES = 4000;

// ---- SASAW (sasaw_segments.hip) ----------------------------------------------
/// Values of a component index that one launch of the matrix-core kernels
/// covers (l <= 3); larger ranges go in parts, a launch per triple of parts,
/// up to SASAW_MAX_PARTS launches, then the general kernels of sasaw.hip.
/// 13 x 7 x 100 components, 900 entries, 60 000 edges: forward 1373 -> 46 us
/// (f32), 1631 -> 105 us (f64) against the general kernel, vjp 3404 -> 862 and
/// 5282 -> 1248 us.
constexpr int SASAW_INDEX_VALUES = 16;
constexpr int32_t SASAW_MAX_PARTS = 64;
/// Rows of W and of grad_output per launch of the gradient kernel when the
/// ranges go in parts: the kernel with 9 accumulator tiles does a row in less
/// than half the time of the one with 16 (13 x 7 x 100 components, 60 000
/// edges, f32: 16 rows 222 us per launch, 9 rows 60 us). In double also the
/// limit for ONE launch on ranges that would fit 16: the 16-tile kernel spills
/// (16 x 16 x 16 components, 64 columns: 950 us in one launch, 784 in four).
constexpr int32_t SASAW_GRADIENT_PART_ROWS = 9;

} // namespace mops::amd::thresholds

#endif
