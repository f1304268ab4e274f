// The rest of Straydog's GPU C ABI: every function the reference's header declares (gpu/straydog_gpu.h, 321 declarations)
// that is not part of the attention path.  The reference's host links the whole library statically and binds all of them
// (crates/straydog-gpu/build.rs:52, crates/straydog-gpu/src/ffi.rs), so an archive that stands in for it must define each
// one.  They fail cleanly, by the ABI's own convention (gpu/straydog_gpu.h:1-5): a negative int or a null pointer, with the
// reason in sd_error(); counts and sizes answer 0; functions without a result do nothing.  A function whose result is text
// never answers null: the host reads such a result as it comes (CStr::from_ptr(ffi::sd_cpu_error()) whenever a CPU-engine call
// has failed, crates/straydog-engine/src/gpu.rs:3831-3838, :3896, :3910; sd_cpu_experts_isa :3928).  sd_cpu_error answers the
// reason the calling thread's last failed call left -- every CPU-engine function here is a stub that leaves one --, any other
// text function its own refusal.
//
// A stub takes no parameters.  In the C calling conventions of the hosts this library is built for (System V x86-64,
// AArch64, Win64) the caller owns the argument area, so a callee that reads none of its arguments is valid whatever the
// caller passed; only the name and the kind of result matter, and abi_stubs.inc lists exactly those.
#include "device.hpp"

namespace {
template<typename Result> Result not_implemented(const char* name, Result result) {
    sd::last_error = std::string(name) + " is not implemented in the attention library";
    return result;
}
// The text a string-returning stub answers: thread-local, so it stays valid until the thread's next failing call.
const char* text_result(const char* name) {
    if (std::strcmp(name, "sd_cpu_error") != 0 || sd::last_error.empty()) (void)not_implemented(name, 0);
    return sd::last_error.c_str();
}
}  // namespace

#define SD_STUB_INT(name) extern "C" int name(void) { return not_implemented(#name, -1); }
#define SD_STUB_PTR(name) extern "C" void* name(void) { return not_implemented(#name, static_cast<void*>(nullptr)); }
#define SD_STUB_STR(name) extern "C" const char* name(void) { return text_result(#name); }
#define SD_STUB_U64(name) extern "C" uint64_t name(void) { return not_implemented(#name, uint64_t(0)); }
#define SD_STUB_I64(name) extern "C" int64_t name(void) { return not_implemented(#name, int64_t(-1)); }
#define SD_STUB_U32(name) extern "C" uint32_t name(void) { return not_implemented(#name, uint32_t(0)); }
#define SD_STUB_VOID(name) extern "C" void name(void) { (void)not_implemented(#name, 0); }

#include "abi_stubs.inc"
