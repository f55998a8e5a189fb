// Internal definitions behind the opaque ACL handles, the executor and the error-message channel.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <vector>

#include "opscv_acl_base.h"

constexpr int kMaxDims = 8;

struct aclTensor {
    int64_t ndim = 0;
    int64_t dims[kMaxDims] = {0};
    int64_t strides[kMaxDims] = {0};  // in elements
    int64_t offset = 0;               // in elements
    aclDataType dtype = ACL_DT_UNDEFINED;
    aclFormat format = ACL_FORMAT_ND;
    int64_t storage_ndim = 0;
    int64_t storage_dims[kMaxDims] = {0};
    void* data = nullptr;

    int64_t numel() const
    {
        int64_t n = 1;
        for (int64_t i = 0; i < ndim; i++) {
            n *= dims[i];
        }
        return n;
    }
    bool empty() const { return numel() == 0; }
    bool contiguous() const
    {
        int64_t expect = 1;
        for (int64_t i = ndim - 1; i >= 0; i--) {
            if (dims[i] != 1 && strides[i] != expect) {
                return false;
            }
            expect *= dims[i];
        }
        return true;
    }
};

struct aclIntArray {
    std::vector<int64_t> v;
};

struct aclFloatArray {
    std::vector<float> v;
};

struct aclBoolArray {
    std::vector<char> v;  // one byte per flag
};

namespace opscv {

enum class Elem : int { F32 = 0, F16 = 1, BF16 = 2 };

inline int elem_size(Elem e) { return e == Elem::F32 ? 4 : 2; }

// dtype -> element kind for the three types the kernels handle; false otherwise
inline bool elem_of(aclDataType dt, Elem* e)
{
    switch (dt) {
        case ACL_FLOAT: *e = Elem::F32; return true;
        case ACL_FLOAT16: *e = Elem::F16; return true;
        case ACL_BF16: *e = Elem::BF16; return true;
        default: return false;
    }
}

// A strided view of up to five dimensions (shorter ones are padded in front with extent 1) that has to be packed
// into (or scattered from) a contiguous workspace slice.
constexpr int kViewDims = 5;
struct StridedView {
    void* base = nullptr;              // tensor data pointer + offset, in bytes
    int64_t dims[kViewDims] = {0};
    int64_t strides[kViewDims] = {0};  // elements
};

enum class OpKind : int { Nop = 0, GridSampler2D = 1, Resize = 2, ResizeGrad = 3, GridSampler3D = 4, GridSampler2DGrad = 5,
                          GridSampler3DGrad = 6 };

// Where a kernel operand lives: the tensor's own memory (contiguous view) or a slice of the caller's
// workspace, known only as an offset until the second phase receives the workspace address.
struct PlannedPtr {
    bool in_workspace = false;
    uint64_t ws_offset = 0;
    void* direct = nullptr;
};

struct GridSamplerArgs {
    Elem elem = Elem::F32;
    int interp = 0;
    int pad = 0;
    int align = 0;
    int channels_last = 0;  // 1: x is (N,Hin,Win,C) and y is (N,Hout,Wout,C) in memory
    // values of the process-wide options (options.hpp) at the time of the first phase:
    int rule = 0;           // bilinear coordinate rule: 0 grid_sampler2_d_simt.h, 1 the arch35 GridSample kernel
    int force_variant = 0;  // GsVariant: 0 automatic choice, 1 direct kernel, 2 no pair-layout variant
    int64_t N = 0, C = 0, Hin = 0, Win = 0, Hout = 0, Wout = 0;
    const void* x = nullptr;
    const void* grid = nullptr;
    void* y = nullptr;
};

// Volumetric sampler: x is (N,C,Din,Hin,Win), grid (N,Dout,Hout,Wout,3) ordered x,y,z, y (N,C,Dout,Hout,Wout).
struct GridSampler3DArgs {
    Elem elem = Elem::F32;
    int interp = 0;  // 0 bilinear (trilinear blend of eight corners), 1 nearest
    int pad = 0;
    int align = 0;
    int channels_last = 0;  // 1: x is (N,Din,Hin,Win,C) and y is (N,Dout,Hout,Wout,C) in memory
    int64_t N = 0, C = 0, Din = 0, Hin = 0, Win = 0, Dout = 0, Hout = 0, Wout = 0;
    const void* x = nullptr;
    const void* grid = nullptr;
    void* y = nullptr;
};

// Backward of the 2-D sampler.  dx / dgrid may be null (output mask): that gradient is then not computed.
struct GridSamplerGradArgs {
    Elem elem = Elem::F32;
    int interp = 0;
    int pad = 0;
    int align = 0;
    int64_t N = 0, C = 0, Hin = 0, Win = 0, Hout = 0, Wout = 0;
    const void* gout = nullptr;  // (N,C,Hout,Wout)
    const void* x = nullptr;     // (N,C,Hin,Win)
    const void* grid = nullptr;  // (N,Hout,Wout,2)
    void* dx = nullptr;          // (N,C,Hin,Win)
    void* dgrid = nullptr;       // (N,Hout,Wout,2)
    // optional scratch of gs2d_grad_csr_words() 32-bit words: the per-element contribution lists of the input
    // gradient (gs2d_grad_csr.hip); null: the input gradient is scattered with elections (gs2d_grad.hip)
    void* scratch = nullptr;
};

// Backward of the 3-D sampler.  dx / dgrid may be null (output mask): that gradient is then not computed.
struct GridSampler3DGradArgs {
    Elem elem = Elem::F32;
    int interp = 0;  // 0 bilinear, 1 nearest
    int pad = 0;
    int align = 0;
    int64_t N = 0, C = 0, Din = 0, Hin = 0, Win = 0, Dout = 0, Hout = 0, Wout = 0;
    int64_t items_per_core = 1;  // batch items the reference walks as one run of grid points (chunk boundaries)
    int force_variant = 0;       // option "gs3d_grad_variant" at the first phase: 0 automatic, 1 ordered kernel, 2 gather
    const void* gout = nullptr;  // (N,C,Dout,Hout,Wout)
    const void* x = nullptr;     // (N,C,Din,Hin,Win)
    const void* grid = nullptr;  // (N,Dout,Hout,Wout,3)
    void* dx = nullptr;          // (N,C,Din,Hin,Win)
    void* dgrid = nullptr;       // (N,Dout,Hout,Wout,3)
    // optional scratch of gs3d_grad_range_words() 32-bit words: the span of voxels every chunk of grid points
    // touches, which lets a band of the input gradient pass over the chunks that miss it; null: every chunk is looked at
    void* chunk_ranges = nullptr;
    // optional scratch of gs3d_grad_list_words() 32-bit words, 16-byte aligned: cell slots and corner weights of the
    // variant that gathers every voxel's contributions (gs3d_grad_lists.hip); null: the ordered kernel does all items
    void* lists = nullptr;
};

enum class ResizeMode : int {
    Bilinear = 0,
    Copy = 1,
    Broadcast = 2,
    FirstPixel = 3,
    Nearest = 4,
    PointCopy = 5,
    FourWeights = 6  // channels-last: sum of four weighted taps instead of two nested blends
};

struct ResizeArgs {
    Elem elem = Elem::F32;
    ResizeMode mode = ResizeMode::Bilinear;
    int half_pixel = 1;
    int channels_last = 0;
    int raw_lambda = 0;  // NCHW bilinear: fraction taken from the unclamped source coordinate (see axis_tap)
    // values of the process-wide options (options.hpp) at the time of the first phase:
    int force_variant = 0;  // ResizeVariant: 0 automatic, 1 per-element kernels, 2 register band, 3 no flat LDS kernel
    int force_nearest = 0;  // NearestVariant: 0 automatic, 1 gather from memory (no LDS staging)
    float scale_h = 1.0f, scale_w = 1.0f;
    int32_t rep_h = 0, rep_w = 0;  // Nearest: whole upscale factors when source = destination / factor is the rule, else 0
    int64_t point_step_h = 1, point_step_w = 1;  // PointCopy: integer source stride per destination pixel
    int64_t N = 0, C = 0, Hs = 0, Ws = 0, Hd = 0, Wd = 0;
    const void* x = nullptr;
    void* y = nullptr;
};

// Backward of the bilinear resize.  "src" is the tensor that was upsampled (the extents of the result `y`), "dst"
// the upsampled one (the extents of the incoming gradient `x`).
struct ResizeGradArgs {
    Elem elem_in = Elem::F32;   // gradient coming in
    Elem elem_out = Elem::F32;  // gradient going out
    int copy = 0;               // equal sizes: y = x
    int user_scales = 0;        // scales that are not the ratio of the sizes: the user-scale template
    int half_pixel = 1;
    int channels_last = 0;
    float scale_h = 1.0f, scale_w = 1.0f, inv_scale_h = 1.0f, inv_scale_w = 1.0f;
    int64_t N = 0, C = 0, Hs = 0, Ws = 0, Hd = 0, Wd = 0;
    const void* x = nullptr;
    void* y = nullptr;
};

}  // namespace opscv

constexpr uint32_t kExecutorMagic = 0x0C5CA11Du;

struct aclOpExecutor {
    uint32_t magic = kExecutorMagic;
    opscv::OpKind kind = opscv::OpKind::Nop;
    uint64_t workspace_bytes = 0;
    opscv::GridSamplerArgs gs;  // pointer members are filled in by the second phase
    opscv::ResizeArgs rs;
    opscv::ResizeGradArgs rg;
    opscv::GridSampler3DArgs gs3;
    opscv::GridSamplerGradArgs gsg;
    opscv::GridSampler3DGradArgs gsg3;
    int want_out0 = 1, want_out1 = 0;  // which outputs the operator produces (backward output mask)
    opscv::PlannedPtr in0, in1, out0;  // input/self, grid, out
    opscv::PlannedPtr in2, out1;       // third input and second output of the operators that have them
    opscv::PlannedPtr scratch;         // kernel scratch inside the workspace (operators that use one)
    // packing work: views gathered into the workspace before the kernel, scattered after it
    struct Pack {
        opscv::StridedView view;
        uint64_t ws_offset = 0;
        int elem_bytes = 0;
    };
    // at most three inputs and two outputs per operator; fixed storage, so that planning never touches the heap
    struct PackList {
        static constexpr int kCapacity = 4;
        Pack items[kCapacity];
        int count = 0;
        // false when the list is full (the entry is dropped: the caller must fail the plan)
        bool push_back(const Pack& p)
        {
            if (count >= kCapacity) {
                return false;
            }
            items[count++] = p;
            return true;
        }
        const Pack* begin() const { return items; }
        const Pack* end() const { return items + count; }
    };
    PackList pack_in;
    PackList unpack_out;
    // a view that needed packing found its list full: the plan is unusable and the first phase reports
    // ACLNN_ERR_INNER (no operator has that many views today; a future one would fail loudly instead of
    // reading an unpacked workspace slice)
    bool pack_overflow = false;
};

namespace opscv {

// printf-style; stores the text for aclGetRecentErrMsg and, when OPSCV_LOG=1, prints it to stderr
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

}  // namespace opscv
