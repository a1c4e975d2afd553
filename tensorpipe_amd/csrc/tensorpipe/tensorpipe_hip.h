// Umbrella header for the GPU side (cf. tensorpipe/tensorpipe_cuda.h of the
// reference): HipBuffer and the three HIP channels, plus the CPU xth channel.
#pragma once

#include <tensorpipe/tensorpipe.h>

#include <tensorpipe/common/hip_buffer.h>

#include <tensorpipe/channel/hip_basic/factory.h>
#include <tensorpipe/channel/hip_ipc/factory.h>
#include <tensorpipe/channel/hip_xth/factory.h>
#include <tensorpipe/channel/xth/factory.h>
