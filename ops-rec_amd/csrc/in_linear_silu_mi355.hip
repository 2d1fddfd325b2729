// C ABI of in_linear_silu forward: argument checks, choice of the kernel variant, launch.  Host-side counterpart of
// the reference's adapter checks (ascendc/activation/in_linear_silu/torch_extension/in_linear_silu_plugin.cpp:36-66)
// and of its host tiling (ascendc/activation/in_linear_silu/in_linear_silu_forward/op_host/in_linear_silu.cpp).
#include "../../include/ops_rec_activation_mi355.h"

#include <hip/hip_runtime.h>

#include "hstu_error.h"
#include "in_linear_silu_bwd_kernel.hip.h"
#include "in_linear_silu_kernel.hip.h"

namespace {

using hstu::InLinearSiluArgs;

struct IlsVariant {
    const char* name;
    void (*kernel)(const InLinearSiluArgs);
    int tile_n;  // output columns per workgroup
};

// [type: bf16, fp16][ring of 2 stages; 3 stages; 4 stages; 2 stages with 128 x 256 tiles].  Measured on MI355X over
// k = 64 .. 8192: for 128 x 128 tiles, workgroups per CU count for more than prefetch depth (4 stages, two workgroups
// per CU, slowest everywhere up to k = 2048); 3 stages win by 3-7 % for k = 128 .. 512, 2 stages by 2-4 % at k <= 64
// and k = 768.  From k = 1024 on the products dominate and the 128 x 256 tile (twice the MFMAs per k step and per byte
// staged, two workgroups per CU) wins: 633 -> 549 us at k = 2048, 607 -> 484 us at m = n = 8192, k = 4096
// (1.14 PFLOP/s).
#define ILS_VARIANT(tag, tagname, S, W) \
    {"in_linear_silu_" tagname "_stages" #S "_tile" #W, hstu::in_linear_silu_kernel<hstu::tag, S, (W) / 64>, W}
const IlsVariant kVariants[2][4] = {
    {ILS_VARIANT(bf16_tag, "bf16", 2, 128), ILS_VARIANT(bf16_tag, "bf16", 3, 128), ILS_VARIANT(bf16_tag, "bf16", 4, 128),
     ILS_VARIANT(bf16_tag, "bf16", 2, 256)},
    {ILS_VARIANT(f16_tag, "f16", 2, 128), ILS_VARIANT(f16_tag, "f16", 3, 128), ILS_VARIANT(f16_tag, "f16", 4, 128),
     ILS_VARIANT(f16_tag, "f16", 2, 256)},
};

const IlsVariant* select(const in_linear_silu_params* p)
{
    int ring;
    if (p->k >= 1024) {
        ring = 3;
    } else {
        ring = (p->k <= 64 || p->k > 512) ? 0 : 1;
    }
    return &kVariants[p->dtype == HSTU_DT_BF16 ? 0 : 1][ring];
}

constexpr int64_t kMinDim = 16;
constexpr int64_t kMaxDim = 512 * 16;

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

// x tiles kept to one XCD each (see the kernel): for a weight matrix of at most 2 MiB -- half an L2 -- with at most 16 n
// tiles per m tile, rows long enough for the x tiles to weigh against the outputs, and at least four groups of m tiles
bool xcd_groups(const in_linear_silu_params* p)
{
    return p->n * p->k * 2 <= (int64_t{2} << 20) && p->n <= 2048 && p->k >= 128 && p->m >= 4096;
}

// workgroups of a launch: m tiles (rounded up to whole groups of one per XCD in the grouped order) times n tiles
int64_t grid_size(const in_linear_silu_params* p)
{
    const int tile_n = select(p)->tile_n;
    int64_t tiles_m = (p->m + hstu::kIlsTileM - 1) / hstu::kIlsTileM;
    const int64_t tiles_n = (p->n + tile_n - 1) / tile_n;
    if (xcd_groups(p)) {
        tiles_m = (tiles_m + hstu::kIlsXcds - 1) / hstu::kIlsXcds * hstu::kIlsXcds;
    }
    return tiles_m * tiles_n;
}

int validate(const in_linear_silu_params* p)
{
    if (p == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(in_linear_silu_params)) {
        return hstu::set_error(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                               sizeof(in_linear_silu_params));
    }
    if (p->x == nullptr || p->weight == nullptr || p->user == nullptr || p->value == nullptr || p->query == nullptr ||
        p->key == nullptr || p->linear_output == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "x, weight and the five outputs must all be given");
    }
    if (p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) {
        return hstu::set_error(HSTU_ERR_INVALID, "dtype %d is not bf16 or fp16", p->dtype);
    }
    if (p->m < 1) {
        return hstu::set_error(HSTU_ERR_INVALID, "x tensor must be non-empty");
    }
    int64_t total = 0;
    for (int i = 0; i < 4; ++i) {
        if (p->split[i] < kMinDim || p->split[i] > kMaxDim || p->split[i] % kMinDim != 0) {
            return hstu::set_error(HSTU_ERR_INVALID, "uvqk dim must in range[16, 8192] and multiples of 16.");
        }
        total += p->split[i];
    }
    if (p->k < kMinDim || p->k > kMaxDim || p->k % kMinDim != 0) {
        return hstu::set_error(HSTU_ERR_INVALID, "x dim[1] must in range[16, 8192] and multiples of 16.");
    }
    if (p->n < 4 * kMinDim || p->n > 4 * kMaxDim || p->n % kMinDim != 0) {
        return hstu::set_error(HSTU_ERR_INVALID, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    }
    if (total != p->n) {
        return hstu::set_error(HSTU_ERR_INVALID, "weight_dim[0] must equal to sum(splitList).");
    }
    if (p->n % (4 * p->k) != 0) {
        return hstu::set_error(HSTU_ERR_INVALID, "weight dim[0] must be a multiple of 4 x dim[1]");
    }
    const void* ptrs[] = {p->x, p->weight, p->bias, p->user, p->value, p->query, p->key, p->linear_output};
    for (const void* ptr : ptrs) {
        if (!aligned16(ptr)) {
            return hstu::set_error(HSTU_ERR_INVALID, "every tensor must start at a multiple of 16 bytes");
        }
    }
    const int64_t tiles = grid_size(p);
    if (tiles > 0x7fffffff) {
        return hstu::set_error(HSTU_ERR_INVALID, "too many rows: %lld tiles of %d rows", static_cast<long long>(tiles),
                               hstu::kIlsTileM);
    }
    return HSTU_OK;
}

int validate_bwd(const in_linear_silu_bwd_params* p)
{
    if (p == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(in_linear_silu_bwd_params)) {
        return hstu::set_error(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                               sizeof(in_linear_silu_bwd_params));
    }
    if (p->linear_output == nullptr || p->user_grad == nullptr || p->value_grad == nullptr || p->query_grad == nullptr ||
        p->key_grad == nullptr || p->d_mixed == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "linear_output, the four gradients and d_mixed must all be given");
    }
    if (p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) {
        return hstu::set_error(HSTU_ERR_INVALID, "dtype %d is not bf16 or fp16", p->dtype);
    }
    if (p->m < 1) {
        return hstu::set_error(HSTU_ERR_INVALID, "linear_output tensor must be non-empty");
    }
    int64_t total = 0;
    for (int i = 0; i < 4; ++i) {
        if (p->split[i] < kMinDim || p->split[i] > kMaxDim || p->split[i] % kMinDim != 0) {
            return hstu::set_error(HSTU_ERR_INVALID, "uvqk dim must in range[16, 8192] and multiples of 16.");
        }
        total += p->split[i];
    }
    if (p->n < 4 * kMinDim || p->n > 4 * kMaxDim || p->n % kMinDim != 0) {
        return hstu::set_error(HSTU_ERR_INVALID, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    }
    if (total != p->n) {
        return hstu::set_error(HSTU_ERR_INVALID, "linear_output dim[1] must equal to sum(split_list).");
    }
    const void* ptrs[] = {p->linear_output, p->user_grad, p->value_grad, p->query_grad, p->key_grad, p->d_mixed};
    for (const void* ptr : ptrs) {
        if (!aligned16(ptr)) {
            return hstu::set_error(HSTU_ERR_INVALID, "every tensor must start at a multiple of 16 bytes");
        }
    }
    if ((p->m + hstu::kIlsBwdRows - 1) / hstu::kIlsBwdRows * ((p->n + hstu::kIlsBwdCols - 1) / hstu::kIlsBwdCols) > 0x7fffffff) {
        return hstu::set_error(HSTU_ERR_INVALID, "too many rows");
    }
    return HSTU_OK;
}

int64_t bwd_row_blocks(const in_linear_silu_bwd_params* p) { return (p->m + hstu::kIlsBwdRows - 1) / hstu::kIlsBwdRows; }

uint64_t bwd_workspace_bytes(const in_linear_silu_bwd_params* p)
{
    return p->bias_grad == nullptr ? 0 : static_cast<uint64_t>(bwd_row_blocks(p)) * static_cast<uint64_t>(p->n) * sizeof(float);
}

}  // namespace

extern "C" {

HSTU_API int in_linear_silu_bwd_dmixed_workspace_size(const in_linear_silu_bwd_params* p, uint64_t* workspace_bytes)
{
    if (workspace_bytes == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "workspace_bytes is NULL");
    }
    *workspace_bytes = 0;
    const int rc = validate_bwd(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    *workspace_bytes = bwd_workspace_bytes(p);
    return HSTU_OK;
}

HSTU_API int in_linear_silu_bwd_dmixed(const in_linear_silu_bwd_params* p, void* workspace, uint64_t workspace_bytes,
                                       void* stream)
{
    const int rc = validate_bwd(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const uint64_t need = bwd_workspace_bytes(p);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))) {
        return hstu::set_error(HSTU_ERR_WORKSPACE, "workspace of %llu bytes (16-byte aligned) needed for the bias gradient, got %llu",
                               static_cast<unsigned long long>(need), static_cast<unsigned long long>(workspace_bytes));
    }
    hstu::InLinearSiluBwdArgs a;
    a.linear_output = p->linear_output;
    a.user_grad = p->user_grad;
    a.value_grad = p->value_grad;
    a.query_grad = p->query_grad;
    a.key_grad = p->key_grad;
    a.d_mixed = p->d_mixed;
    a.partial_sums = need > 0 ? static_cast<float*>(workspace) : nullptr;
    a.m = p->m;
    a.n = static_cast<int>(p->n);
    a.split_end[0] = static_cast<int>(p->split[0]);
    a.split_end[1] = a.split_end[0] + static_cast<int>(p->split[1]);
    a.split_end[2] = a.split_end[1] + static_cast<int>(p->split[2]);
    const unsigned col_blocks = static_cast<unsigned>((p->n + hstu::kIlsBwdCols - 1) / hstu::kIlsBwdCols);
    const unsigned row_blocks = static_cast<unsigned>(bwd_row_blocks(p));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (p->dtype == HSTU_DT_BF16) {
        hipLaunchKernelGGL(hstu::in_linear_silu_dmixed_kernel<hstu::bf16_tag>, dim3(row_blocks * col_blocks),
                           dim3(hstu::kIlsBwdThreads), 0, s, a);
    } else {
        hipLaunchKernelGGL(hstu::in_linear_silu_dmixed_kernel<hstu::f16_tag>, dim3(row_blocks * col_blocks),
                           dim3(hstu::kIlsBwdThreads), 0, s, a);
    }
    if (need > 0) {
        hipLaunchKernelGGL(hstu::in_linear_silu_bias_grad_kernel,
                           dim3(static_cast<unsigned>((p->n + hstu::kIlsBiasCols - 1) / hstu::kIlsBiasCols)),
                           dim3(hstu::kIlsBiasCols * hstu::kIlsBiasLanes), 0, s, a.partial_sums, p->bias_grad,
                           static_cast<int>(row_blocks), a.n);
    }
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return hstu::set_error(HSTU_ERR_RUNTIME, "launch of in_linear_silu_dmixed failed: %s", hipGetErrorString(err));
    }
    return HSTU_OK;
}

HSTU_API const char* in_linear_silu_fwd_kernel_name(const in_linear_silu_params* params)
{
    return validate(params) == HSTU_OK ? select(params)->name : nullptr;
}

HSTU_API int in_linear_silu_fwd(const in_linear_silu_params* p, void* stream)
{
    const int rc = validate(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const IlsVariant* v = select(p);
    InLinearSiluArgs a;
    a.x = p->x;
    a.weight = p->weight;
    a.bias = p->bias;
    a.user = p->user;
    a.value = p->value;
    a.query = p->query;
    a.key = p->key;
    a.linear_output = p->linear_output;
    a.m = p->m;
    a.n = static_cast<int>(p->n);
    a.k = static_cast<int>(p->k);
    a.split_end[0] = static_cast<int>(p->split[0]);
    a.split_end[1] = a.split_end[0] + static_cast<int>(p->split[1]);
    a.split_end[2] = a.split_end[1] + static_cast<int>(p->split[2]);
    a.xcd_groups = xcd_groups(p) ? 1 : 0;
    const int64_t tiles = grid_size(p);
    hipLaunchKernelGGL(v->kernel, dim3(static_cast<unsigned>(tiles)), dim3(hstu::kIlsThreads), 0,
                       static_cast<hipStream_t>(stream), a);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return hstu::set_error(HSTU_ERR_RUNTIME, "launch of %s failed: %s", v->name, hipGetErrorString(err));
    }
    return HSTU_OK;
}

}  // extern "C"
