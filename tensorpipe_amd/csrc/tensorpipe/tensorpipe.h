// Umbrella header (cf. tensorpipe/tensorpipe.h of the reference): core API,
// the shm transport and the CPU channels.
#pragma once

#include <tensorpipe/common/buffer.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/device.h>
#include <tensorpipe/common/error.h>
#include <tensorpipe/common/optional.h>

#include <tensorpipe/core/context.h>
#include <tensorpipe/core/error.h>
#include <tensorpipe/core/listener.h>
#include <tensorpipe/core/message.h>
#include <tensorpipe/core/pipe.h>

#include <tensorpipe/transport/context.h>
#include <tensorpipe/transport/error.h>
#include <tensorpipe/transport/shm/factory.h>
#include <tensorpipe/transport/tcp/factory.h>
#include <tensorpipe/transport/shm_stock/factory.h>

#include <tensorpipe/channel/context.h>
#include <tensorpipe/channel/error.h>
#include <tensorpipe/channel/basic/factory.h>
