// Symbol visibility for the nz:: host library (counterpart of the reference's
// include/NeuZephyr/dl_export.cuh:4-13).
#ifndef NZ_DL_EXPORT_CUH
#define NZ_DL_EXPORT_CUH
#if defined(_WIN32)
#error "the MI355X build targets Linux/ROCm only"
#endif
#define DL_API __attribute__((visibility("default")))
#endif
