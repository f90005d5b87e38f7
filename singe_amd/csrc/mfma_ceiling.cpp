// Host side of the register-only product loop (mfma_ceiling.hip): a measurement aid with no counterpart in the
// reference, whose tuning code times its own kernels the same way (kernel_tuning/measure/mod.rs:34-53).
#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"

using namespace singe_hip;

extern "C" int32_t singe_hip_hbm_stream_read(void* stream, const void* data, size_t bytes, uint32_t* out, size_t out_len,
                                             uint32_t workgroups) {
    if (data == nullptr) return fail(SINGE_HIP_NULL_POINTER, "data");
    if (out == nullptr) return fail(SINGE_HIP_NULL_POINTER, "out");
    if (workgroups == 0) return fail(SINGE_HIP_INVALID_LENGTH, "workgroups");
    if (bytes < 16) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "data", 16, bytes);
    const size_t lanes = static_cast<size_t>(workgroups) * 512;
    if (out_len < lanes) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "out", lanes, out_len);
    HbmStreamArgs args;
    args.data = data;
    args.out = out;
    args.chunks = bytes / 16;
    return launch(kHbmStreamRead, workgroups, 1, 1, 512, stream, args);
}

extern "C" int32_t singe_hip_mfma_ceiling(void* stream, const void* operands, size_t operand_bytes, float* out, size_t out_len,
                                          uint32_t workgroups, uint32_t iterations, int32_t f16) {
    if (operands == nullptr) return fail(SINGE_HIP_NULL_POINTER, "operands");
    if (out == nullptr) return fail(SINGE_HIP_NULL_POINTER, "out");
    if (workgroups == 0 || iterations == 0) return fail(SINGE_HIP_INVALID_LENGTH, "workgroups or iterations");
    if (operand_bytes < 16) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "operands", 16, operand_bytes);
    const size_t lanes = static_cast<size_t>(workgroups) * 256;
    if (out_len < lanes) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "out", lanes, out_len);
    MfmaCeilingArgs args;
    args.operands = operands;
    args.out = out;
    args.operand_chunks = operand_bytes / 16;
    args.iterations = iterations;
    return launch(f16 ? kMfmaCeilingF16 : kMfmaCeilingBf16, workgroups, 1, 1, 256, stream, args);
}
