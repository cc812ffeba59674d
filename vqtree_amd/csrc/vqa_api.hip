// Version and error strings of libvqattn.
#include "vqa_common.h"

extern "C" {

int vqa_version(void) { return 110; /* 0.1.1: vqa_decode_roped_*, window kinds of the pipelined core */ }

const char* vqa_strerror(int status) {
    switch (status) {
        case VQA_OK: return "ok";
        case VQA_ERR_NULL_POINTER: return "a required pointer argument is null";
        case VQA_ERR_BAD_SHAPE: return "bad tensor shape (non-positive or inconsistent sizes)";
        case VQA_ERR_UNSUPPORTED_HEAD_DIM: return "unsupported head dimension (supported: 64, 128)";
        case VQA_ERR_UNSUPPORTED_CODEBOOK: return "unsupported codebook configuration (M in {1,2,4,8}, K <= 256)";
        case VQA_ERR_MISALIGNED: return "pointer or stride violates the alignment the kernels need";
        case VQA_ERR_WORKSPACE_TOO_SMALL: return "workspace is smaller than the *_workspace_bytes query reports";
        case VQA_ERR_BAD_ARGUMENT: return "argument out of range";
        case VQA_ERR_LAUNCH_FAILED: return "HIP kernel launch failed";
        case VQA_ERR_SCRATCH_LIMIT:
            return "problem needs more scratch than the static array of the allocation-free entry point holds";
        default: return "unknown vqa status";
    }
}

}  // extern "C"
