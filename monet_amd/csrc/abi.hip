// ABI bookkeeping entry points of libmonet_hip.so.
#include "common.h"

extern "C" {

int mn_abi_version(void) { return 1; }

int mn_init(void) {
  const bool bn = mn_bn_static_init(), wino = mn_wino_init();
  return bn && wino ? MN_OK : MN_ELAUNCH;
}

const char* mn_status_string(int status) {
  switch (status) {
    case MN_OK:
      return "ok";
    case MN_EINVAL:
      return "invalid argument (null pointer, bad size, misaligned operand or workspace too small)";
    case MN_EUNSUPPORTED:
      return "unsupported shape, variant or dtype";
    case MN_ELAUNCH:
      return "kernel launch failed, or a kernel reported that it could not finish its work";
    case MN_ELIMIT:
      return "the call needs more than a fixed limit of this entry point allows";
    default:
      return "unknown status";
  }
}

}  // extern "C"
