// Internal definitions behind the opaque aclTensor / aclOpExecutor handles.
#pragma once
#include <cstdarg>
#include <cstdint>
#include <string>
#include <vector>

#include "acl/acl.h"
#include "opsnn_kernels.h"

struct aclTensor {
    std::vector<int64_t> view;     // view shape, in elements
    std::vector<int64_t> strides;  // in elements
    int64_t offset = 0;            // in elements
    aclDataType dtype = ACL_DT_UNDEFINED;
    aclFormat format = ACL_FORMAT_ND;
    std::vector<int64_t> storage;  // storage shape
    void* data = nullptr;
};

namespace opsnn {

constexpr uint32_t kExecutorMagic = 0x51454D4Du;

enum class OpKind { None, QmmInt8, QmmBlockScale, QmmMx, QmmTc, QmmGroup, Wqmm, DynQuant, BlockQuant, MxQuant, TransQuantParam, Prepack };

// What phase 1 decided; phase 2 only fills in workspace/stream and launches.
struct aclOpExecutorImpl {
    uint32_t magic = kExecutorMagic;
    OpKind kind = OpKind::None;     // None: nothing to launch (empty output)
    OpsnnQmmArgs qmm{};
    OpsnnWqmmArgs wqmm{};
    OpsnnDynQuantArgs dynq{};
    OpsnnBlockQuantArgs blkq{};
    OpsnnMxQuantArgs mxq{};
    struct { const float* scale; int64_t scale_len; const float* offset; int64_t offset_len; int round_mode; uint64_t* out; } tqp{};
    // aclnnPrepackMatmulWeight: [batch, k, n] -> [batch, n, k] of `bits`-wide elements (src in ND, or in FRACTAL_NZ via `nz`),
    // and optionally a 16-bit scale matrix [batch, srows, scols] -> [batch, scols, srows]
    struct { const void* src; void* dst; int64_t k, n, batch; int bits; const void* ssrc; void* sdst; int64_t srows, scols, sbatch; } prepack{};
    uint64_t workspace_size = 0;
    const char* api = "";
    // Right operand handed over in FRACTAL_NZ (the ...WeightNz / ...Nz entry points): phase 2 first re-lays it out as the
    // dense ND matrix into the front of the workspace (nd_bytes, rounded up to 256), points the operand there, and gives
    // the rest of the workspace to the launcher.
    // General batch broadcast of aclnnQuantMatmulV5 (x1 [2, 1, M, K] with x2 [1, 3, K, N] and the like): one launch per
    // combination of the outer batch dims, each over the innermost batch dim; empty for the usual cases, which are one launch.
    std::vector<OpsnnQmmArgs> batch_runs;
    // Strided view of a 4-bit matrix operand, or of an 8-bit one in the MX modes (index 0: x1, 1: x2): phase 2 first gathers it
    // into a dense copy at the very front of the workspace (bytes, rounded up to 256, each) and points the operand there.
    struct GatherStep { bool active = false; int bits = 4; const void* base = nullptr; int64_t off = 0, nb = 1, rows = 0, cols = 0, bs = 0, rs = 0, cs = 0; uint64_t bytes = 0; } gather[2];
    uint64_t gather_front() const { return (gather[0].active ? (gather[0].bytes + 255) / 256 * 256 : 0) + (gather[1].active ? (gather[1].bytes + 255) / 256 * 256 : 0); }
    struct NzStep { bool active = false; const void* src = nullptr; int64_t rows = 0, row_bytes = 0, batch = 1; int c0 = 0; uint64_t nd_bytes = 0; } nz;
};

// Live executors.  Phase 1 hands an executor over with executor_publish(); phase 2 and aclDestroyAclOpExecutor take it
// back with executor_claim(), which succeeds once per published pointer.  A handle that was already run or destroyed
// is recognised by its absence from the set, without reading through the (freed) pointer.
struct aclOpExecutorImpl;
void* executor_publish(void* ex);
bool executor_claim(const void* ex);

// Thread-local last-error text (aclGetRecentErrMsg).
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();
bool log_enabled();

inline bool is_4bit(aclDataType d) { return d == ACL_INT4 || d == ACL_FLOAT4_E2M1 || d == ACL_FLOAT4_E1M2; }
inline int dtype_bits(aclDataType d)
{
    switch (d) {
        case ACL_FLOAT: case ACL_INT32: case ACL_UINT32: return 32;
        case ACL_FLOAT16: case ACL_BF16: case ACL_INT16: case ACL_UINT16: return 16;
        case ACL_INT8: case ACL_UINT8: case ACL_BOOL: case ACL_HIFLOAT8: case ACL_FLOAT8_E5M2:
        case ACL_FLOAT8_E4M3FN: case ACL_FLOAT8_E8M0: return 8;
        case ACL_INT64: case ACL_UINT64: case ACL_DOUBLE: case ACL_COMPLEX64: return 64;
        case ACL_INT4: case ACL_FLOAT4_E2M1: case ACL_FLOAT4_E1M2: return 4;
        default: return 0;
    }
}
const char* dtype_name(aclDataType d);
std::string shape_str(const std::vector<int64_t>& s);

// A lightweight copy of a tensor's view that the checks may rewrite (swap dims, re-tag dtype).
struct TView {
    std::vector<int64_t> shape, strides;
    int64_t offset = 0;
    aclDataType dtype = ACL_DT_UNDEFINED;
    aclFormat format = ACL_FORMAT_ND;
    std::vector<int64_t> storage;
    void* data = nullptr;
    bool present = false;
    int64_t rank() const { return (int64_t)shape.size(); }
    int64_t dim(int64_t i) const { return shape[(size_t)(i < 0 ? i + rank() : i)]; }
    int64_t stride(int64_t i) const { return strides[(size_t)(i < 0 ? i + rank() : i)]; }
    int64_t numel() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
    bool empty() const { return numel() == 0; }
    // address of element offset `off` (in elements) from the storage base
    const void* ptr_at(int64_t off) const
    {
        if (!data) return nullptr;
        return (const char*)data + ((offset + off) * dtype_bits(dtype)) / 8;
    }
};
TView make_view(const aclTensor* t);
bool is_contiguous(const TView& v);
// Last two dims transposed: stride[-2]==1, stride[-1]==shape[-2], dense batch strides, not both extents 1.
bool is_transposed_last2(const TView& v);
void swap_last2(TView& v);

// Phase 1 helper: checks the FRACTAL_NZ storage shape [.., ceil(cols / c0), ceil(rows / 16), 16, c0] of a right operand whose
// stored matrix is [.., rows, cols] (the view, or its last two dims swapped for a transposed view) and fills the step.
// Returns false with the error text set.
bool describe_nz_operand(const char* api, const char* name, const aclTensor* t, aclOpExecutorImpl::NzStep* step);
// Phase 2 helper for executors with an NZ pre-step: runs it, returns the ND operand's address and the rest of the workspace.
int run_nz_step(const aclOpExecutorImpl& ex, void* workspace, void* stream, const void** nd_ptr, void** rest);
inline uint64_t nz_front_bytes(const aclOpExecutorImpl& ex) { return ex.nz.active ? (ex.nz.nd_bytes + 255) / 256 * 256 : 0; }

}  // namespace opsnn

struct aclOpExecutor : opsnn::aclOpExecutorImpl {};
