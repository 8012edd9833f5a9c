// Test infrastructure: stands in for the HIP runtime header when a kernel source is compiled for the host; everything
// the sources use comes from the stand-in ovl_device.h of this directory.
#ifndef OVL_HOST_EMULATION_HIP_RUNTIME_H_
#define OVL_HOST_EMULATION_HIP_RUNTIME_H_
#endif
