// rtc.hpp -- round kernels for a statement generated at run time.  The reference compiles a kernel for any
// statement on first use (ROUND-KERNEL, src/sumcheck.lisp:260-280); here the statement's descriptor becomes a
// compile-time constant of the same kernel templates the build instantiates for the listed statements, compiled
// through hiprtc on background threads while the interpreter kernel serves the statement, and loaded into the
// registry of generated kernels once the code is there.
#pragma once
#include <string>

#include "stmtdesc.hpp"

namespace exh {

// false when EXACTA_HIP_NO_RTC is set
bool rtc_enabled();
// Start compiling kernels for the planned statement (its key, descriptor and degree D) unless that was done or
// asked before.  Returns at once.
// `source` (optional): the text of `struct RtStmt` when it is more than the descriptor (a statement in direct form).
void rtc_request(const std::string &key, const StmtDesc &desc, int D, const std::string &source = std::string());
// Load the compilations that have finished into the registry.  Called by the thread that owns the device,
// before it looks a statement up.  Returns E_DEVICE when a module does not load.
int rtc_collect();
// 1: kernels for (key, D) are registered; 0: their compilation is still running (or was never asked for);
// E_DEVICE with the compiler's log as the error text when it failed.  With wait, blocks until it has ended.
int rtc_status(const std::string &key, int D, bool wait);
// 1 when no compilation is running (with wait: once none is, their kernels loaded), 0 while one runs
int rtc_idle(bool wait);

}  // namespace exh
