// The symbol NCCL/RCCL looks up after dlopen("libnccl-net.so"): the version-7 function table, in the member order
// and with the name string of the reference (src/nccl_plugin.cc:22-42).
#include "tcpx_plugin.h"

extern "C" {

volatile ncclNet_v7_t ncclNetPlugin_v7 = {
    "GPUDirectTCPX_v7",
    tcpxInit,
    tcpxDevices,
    tcpxGetProperties,
    tcpxListen,
    tcpxConnect_v5,
    tcpxAccept_v5,
    tcpxRegMr,
    nullptr,  // regMrDmaBuf: not provided, as in the reference
    tcpxDeregMr,
    tcpxIsend_v5,
    tcpxIrecv_v5,
    tcpxIflush_v5,
    tcpxTest,
    tcpxClose,  // closeSend
    tcpxClose,  // closeRecv
    tcpxCloseListen,
    tcpxGetDeviceMr,
    tcpxIrecvConsumed,
};

}
