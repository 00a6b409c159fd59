/*
 * nccl_net_v7.h -- the slice of the NCCL network-plugin ABI (version 7) that the receive-side unpack path
 * touches, declared here because no NCCL/RCCL development headers ship with this build.
 *
 * The reference (google/nccl-plugin-gpudirecttcpx) compiles against NCCL's nccl.h, nccl_net.h, net_device.h
 * and unpack_defs.h; the names, field orders and values below are fixed by how the reference uses them:
 *   result codes                          src/adapter/nccl/ret.h:22-31, src/adapter/native/ret.h:21-29
 *   ncclNetProperties_v7_t fields         src/net_tcpx.cc:725-744
 *   ncclNetDeviceHandle_v7_t fields       src/net_tcpx.cc:1463-1467
 *   ncclNet_v7_t member order             src/nccl_plugin.cc:22-42, signatures src/net_tcpx.h:22-62
 *   loadMeta / netUnpackMeta / handle     src/sock/tcpx.h:178-180, src/devcomm/nccl/unpack1.h:52-53,
 *                                         src/devcomm/nccl/unpack1.cu:53-63
 *   queue depth 16, 2048 pages per slot   src/devcomm/nccl/unpack_defs1.h:22-23, src/net_tcpx.cc:1350
 *   logger call shape                     src/adapter/nccl/debug.h:25-35
 * A plugin built from this header is loaded by NCCL/RCCL through the symbol `ncclNetPlugin_v7`.
 */
#ifndef TCPX_AMD_NCCL_NET_V7_H_
#define TCPX_AMD_NCCL_NET_V7_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  ncclSuccess = 0,
  ncclUnhandledCudaError = 1,
  ncclSystemError = 2,
  ncclInternalError = 3,
  ncclInvalidArgument = 4,
  ncclInvalidUsage = 5,
  ncclRemoteError = 6,
  ncclInProgress = 7,
  ncclNumResults = 8
} ncclResult_t;

typedef enum {
  NCCL_LOG_NONE = 0,
  NCCL_LOG_VERSION = 1,
  NCCL_LOG_WARN = 2,
  NCCL_LOG_INFO = 3,
  NCCL_LOG_ABORT = 4,
  NCCL_LOG_TRACE = 5
} ncclDebugLogLevel;

/* Subsystem bits passed as `flags` to the logger. */
#define NCCL_INIT 0x1ul
#define NCCL_NET 0x10ul
#define NCCL_ALL (~0ul)

typedef void (*ncclDebugLogger_t)(ncclDebugLogLevel level, unsigned long flags, const char* file, int line,
                                  const char* fmt, ...);

#define NCCL_PTR_HOST 0x1
#define NCCL_PTR_CUDA 0x2 /* device memory; the name is NCCL's */
#define NCCL_NET_HANDLE_MAXSIZE 128

typedef enum { NCCL_NET_DEVICE_HOST = 0, NCCL_NET_DEVICE_UNPACK = 1 } ncclNetDeviceType;
#define NCCL_NET_DEVICE_INVALID_VERSION 0x0
#define NCCL_NET_DEVICE_UNPACK_VERSION 0x7

typedef struct {
  ncclNetDeviceType netDeviceType;
  int netDeviceVersion;
  void* handle; /* device memory: struct unpackNetDeviceHandle */
  size_t size;
  int needsProxyProgress;
} ncclNetDeviceHandle_v7_t;

typedef struct {
  char* name;
  char* pciPath;
  uint64_t guid;
  int ptrSupport;
  int speed; /* Mb/s */
  int port;
  float latency;
  int maxComms;
  int maxRecvs;
  ncclNetDeviceType netDeviceType;
  int netDeviceVersion;
} ncclNetProperties_v7_t;

typedef struct {
  const char* name;
  ncclResult_t (*init)(ncclDebugLogger_t logFunction);
  ncclResult_t (*devices)(int* ndev);
  ncclResult_t (*getProperties)(int dev, ncclNetProperties_v7_t* props);
  ncclResult_t (*listen)(int dev, void* handle, void** listenComm);
  ncclResult_t (*connect)(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v7_t** sendDevComm);
  ncclResult_t (*accept)(void* listenComm, void** recvComm, ncclNetDeviceHandle_v7_t** recvDevComm);
  ncclResult_t (*regMr)(void* comm, void* data, int size, int type, void** mhandle);
  ncclResult_t (*regMrDmaBuf)(void* comm, void* data, size_t size, int type, uint64_t offset, int fd, void** mhandle);
  ncclResult_t (*deregMr)(void* comm, void* mhandle);
  ncclResult_t (*isend)(void* sendComm, void* data, int size, int tag, void* mhandle, void** request);
  ncclResult_t (*irecv)(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request);
  ncclResult_t (*iflush)(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request);
  ncclResult_t (*test)(void* request, int* done, int* sizes);
  ncclResult_t (*closeSend)(void* sendComm);
  ncclResult_t (*closeRecv)(void* recvComm);
  ncclResult_t (*closeListen)(void* listenComm);
  ncclResult_t (*getDeviceMr)(void* comm, void* mhandle, void** dptr_mhandle);
  ncclResult_t (*irecvConsumed)(void* recvComm, int n, void* request);
} ncclNet_v7_t;

/* ---- unpack metadata shared between the plugin (producer) and the GPU consumer -------------------------- */

#define NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH 16
#define NET_UNPACK_MAX_SLICE_SIZE 4194304
#define SLICE_PAGE_SIZE 4096
#define NET_UNPACK_MAX_SLICE_PAGES (NET_UNPACK_MAX_SLICE_SIZE / SLICE_PAGE_SIZE * 2) /* 2048 */

#ifdef __cplusplus
union alignas(16) loadMeta {
#else
union loadMeta {
#endif
  uint64_t r64[2];
  struct {
    uint32_t src_off; /* from the bounce buffer base */
    uint32_t len;
    uint64_t dst_off; /* from the request's receive buffer */
  };
};

struct netUnpackMeta {
  union loadMeta mem[NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH][NET_UNPACK_MAX_SLICE_PAGES];
  uint64_t cnt[NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH];
};

struct unpackNetDeviceHandle {
  struct netUnpackMeta* meta; /* device alias of the mapped metadata */
  void* bounce_buf;           /* device address of the bounce arena */
  uint64_t head;
};

#ifdef __cplusplus
}
static_assert(sizeof(union loadMeta) == 16, "loadMeta is 16 bytes");
static_assert(sizeof(struct netUnpackMeta) == 16 * 2048 * 16 + 16 * 8, "netUnpackMeta layout");
static_assert(sizeof(struct unpackNetDeviceHandle) == 24, "unpackNetDeviceHandle is 24 bytes");
#endif
#endif /* TCPX_AMD_NCCL_NET_V7_H_ */
