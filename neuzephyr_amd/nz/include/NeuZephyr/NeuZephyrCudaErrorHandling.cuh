// Error type raised when the device runtime reports a failure. Same class name, fields and
// message layout as the reference (include/NeuZephyr/NeuZephyrCudaErrorHandling.cuh:63-106) so
// that `catch (nz::CudaException&)` keeps working; the code carried is a hipError_t (or a
// negative NZHIP_E_* status) and, unlike the reference's CHECK macro (:108-115), the device is
// NOT reset before throwing.
#ifndef NZ_ERROR_HANDLING_CUH
#define NZ_ERROR_HANDLING_CUH
#include <cstdio>
#include <stdexcept>
#include <string>

#include "dl_export.cuh"

namespace nz {
    class DL_API CudaException final : public std::runtime_error {
    public:
        CudaException(const char* file, int line, int code, const char* expr, const char* text)
            : std::runtime_error(text ? text : "device runtime error"), file(file), line(line), code(code), expr(expr) {
            char buffer[1024];
            snprintf(buffer, sizeof(buffer),
                     "HIP Exception:\n\tFile:       %s\n\tLine:       %d\n\tError code: %d\n\tError text: %s\n\tExpression: %s",
                     file, line, code, std::runtime_error::what(), expr);
            msg = buffer;
        }
        const char* what() const noexcept override { return msg.c_str(); }
        int errorCode() const noexcept { return code; }

    private:
        const char* file;
        int line;
        int code;
        const char* expr;
        std::string msg;
    };

    namespace detail {
        // Maps a C-ABI status to the exception the reference API would raise.
        DL_API void throwStatus(int status, const char* file, int line, const char* expr);
    }
}

#define NZ_CHECK(call)                                                            \
    do {                                                                          \
        const int nz_status__ = (call);                                           \
        if (nz_status__ != 0) nz::detail::throwStatus(nz_status__, __FILE__, __LINE__, #call); \
    } while (0)
#endif
