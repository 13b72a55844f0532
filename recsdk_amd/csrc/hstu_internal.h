// Internal declarations shared by the C-ABI translation unit and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <mutex>

#include "../../include/hstu_hip.h"

namespace hstu {

// records the message hstu_hip_last_error() returns to the calling thread; returns `code`
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// private bit of hstu_fwd_params.flags inside the library (callers' copies of it are cleared): every Q tile stays one
// item, no K ranges with partial sums
constexpr uint32_t FLAG_WHOLE_TILES = 0x80000000u;

enum OpKind : int32_t { OP_JAGGED = 0, OP_PAGED = 1, OP_DENSE = 2 };

// Kernel argument block: the caller's parameters plus what the host derives from them.
struct KArgs {
    hstu_fwd_params p;
    int32_t op;          // OpKind
    int32_t head_ratio;  // heads_q / heads_k
    float out_scale;     // factor applied once to the fp32 accumulator (MFMA kernels)
    float exp_scale;     // -alpha * log2(e) (MFMA kernels)
};

// launchers (defined next to their kernels); return hipError_t of the launch
hipError_t launch_generic(const KArgs& a, hipStream_t stream);
bool mfma_supported(const KArgs& a, const char** name);
// bytes of device workspace the MFMA path needs for its work list; the buffer needs no initialisation
uint64_t mfma_workspace_bytes(const KArgs& a);
hipError_t launch_mfma(const KArgs& a, void* workspace, hipStream_t stream);
// the call runs without a schedule kernel: the workgroups of the main kernel derive their items from the offsets
bool mfma_self_scheduled(const KArgs& a);
// the same three for float8_e4m3fn q / k / v (reached through the three above)
bool mfma_fp8_supported(const KArgs& a, const char** name);
uint64_t mfma_fp8_workspace_bytes(const KArgs& a);
hipError_t launch_mfma_fp8(const KArgs& a, void* workspace, hipStream_t stream);
bool mfma_fp8_self_scheduled(const KArgs& a);

// The device-built work list of the MFMA kernels, for kernels outside hstu_mfma.hip.  Layout (uint32 words): 16 header
// words ([2..3] = rows the sequences own, int64), then `grid` records of 8 words, read by workgroup index:
// seq | head << 12 | tile << 16 | sweep << 24 | further tiles << 25 | 1 << 28, then q_start, lq, k_start, lk,
// num_context, num_target, first page entry of the sequence; 0xffffffff in word 0 = no work.  `sweep`: the item also
// covers every later tile of its sequence (rows behind the max_seq_len attribute).
struct WorkList {
    unsigned grid;     // workgroups to launch = records
    uint64_t bytes;    // workspace bytes of the list
};
constexpr unsigned WORK_ITEM_EMPTY = 0xffffffffu;
constexpr int WORK_HEADER_WORDS = 16, WORK_RECORD_WORDS = 8;
WorkList work_list_shape(const hstu_fwd_params& p);
hipError_t launch_work_list(const KArgs& a, unsigned* ws, bool pair, hipStream_t stream);
// dV of the backward as a forward pass over reversed rows (head dim 128, plain causal self-attention without GQA):
// `a` carries K as q, Q as k, dO as v and dV as out; `ws` is a list launch_work_list() built for the same geometry.
// Two streams and three events of the library's own for entry points that run independent kernels side by side: forked from
// and joined to the caller's stream by the events, so that the call stays one piece of work on that stream (also under stream
// capture).  Default priority, events without timing.  Every caller stream gets a set of its own (up to 8 per device, made
// at the stream's first such call; further streams share the last set), so that host threads on streams of their own do
// not queue up behind one pair of side streams.  A call holds the set's mutex from its first event record to its last
// wait (these only enqueue work).  nullptr: run on the caller's stream -- HSTU_HIP_SERIAL_BACKWARD=1 is set, or the set
// could not be made (tried again at the next call, three times per set; never while the caller's stream is capturing,
// since creating streams may not be legal then).
struct SideStreams {
    hipStream_t side[2];
    hipEvent_t ev[3];
    std::mutex mu;
};
SideStreams* side_streams(hipStream_t caller);
bool reversed_forward_supported(const hstu_fwd_params& p);
hipError_t launch_reversed_forward(const KArgs& a, const unsigned* ws, hipStream_t stream);

// Backward of the jagged op: the forward's argument block plus the gradient buffers.
struct BArgs {
    KArgs f;
    const void* grad_out;
    void* grad_q;
    void* grad_k;
    void* grad_v;
    void* grad_bias;
};
hipError_t launch_backward_generic(const BArgs& a, hipStream_t stream);
bool mfma_backward_supported(const BArgs& a);
uint64_t mfma_backward_workspace_bytes(const BArgs& a);
hipError_t launch_backward_mfma(const BArgs& a, void* workspace, hipStream_t stream);

}  // namespace hstu
