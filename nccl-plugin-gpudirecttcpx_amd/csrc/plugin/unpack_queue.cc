// The unpack-metadata queue of one comm: mapped host memory holding NCCL's netUnpackMeta plus the completion
// words, a 24-byte device handle, and the host-side head/tail/record (src/devcomm/nccl/unpack1.cu:28-86,
// src/devcomm/nccl/unpack1.h:30-65).
#include "plugin_internal.h"

namespace tcpx {

ncclResult_t unpack_queue_new(int dev, bool passive, UnpackQueue** queue) {
  DeviceState* ds = &g.devices[dev];
  UnpackQueue* q = new (std::nothrow) UnpackQueue;
  if (!q) return ncclSystemError;
  q->dev = dev;
  memset(&q->record, 0, sizeof q->record);
  QueueBlock blk{};
  {
    std::lock_guard<std::mutex> lock(ds->mu);
    if (!ds->free_blocks.empty()) {
      blk = ds->free_blocks.back();
      ds->free_blocks.pop_back();
    }
  }
  if (!blk.meta) {
    void *h = nullptr, *d = nullptr, *dh = nullptr;
    ncclResult_t rc = device_result(g.ops->mapped_alloc(dev, sizeof(QueueMeta), &h, &d), "mapped_alloc");
    if (rc == ncclSuccess) rc = device_result(g.ops->device_alloc(dev, sizeof(struct unpackNetDeviceHandle), &dh),
                                              "device_alloc");
    if (rc != ncclSuccess) {
      delete q;
      return rc;
    }
    void *sh = nullptr, *sd = nullptr;
    if (!g.ops->visible_alloc || !g.ops->visible_flush ||
        g.ops->visible_alloc(dev, sizeof(union loadMeta) * kStagedDescs * kQueueDepth, &sh, &sd) != TCPXU_SUCCESS) {
      sh = sd = nullptr;  // optional: every request's descriptors are then read from the mapped slot
    }
    blk = QueueBlock{static_cast<QueueMeta*>(h), static_cast<QueueMeta*>(d),
                     static_cast<struct unpackNetDeviceHandle*>(dh), static_cast<union loadMeta*>(sh),
                     static_cast<union loadMeta*>(sd)};
  }
  memset(blk.meta, 0, sizeof(QueueMeta));
  q->meta = blk.meta;
  q->meta_dev = blk.meta_dev;
  q->dev_handle = blk.dev_handle;
  q->stage = blk.stage;
  q->stage_dev = blk.stage_dev;
  // Device-side handle {meta, bounce_buf, head}; head starts at -1 because NCCL's consumer increments it before
  // it copies (src/devcomm/nccl/unpack1.cu:54-63).  Only the receiving side knows a bounce buffer.
  struct unpackNetDeviceHandle hd;
  hd.meta = &q->meta_dev->nccl;
  hd.bounce_buf = passive ? ds->arena : nullptr;
  hd.head = static_cast<uint64_t>(-1);
  ncclResult_t rc = device_result(g.ops->copy_to_device(dev, q->dev_handle, &hd, sizeof hd), "copy_to_device");
  if (rc != ncclSuccess) {
    unpack_queue_free(q);
    return rc;
  }
  *queue = q;
  return ncclSuccess;
}

void unpack_queue_free(UnpackQueue* q) {
  if (!q) return;
  // Mapped and device memory cannot be released while the persistent kernel runs (the runtime waits for every
  // stream of the device when it frees), so the block goes back to the device's pool; tcpxFinalize releases it.
  DeviceState* ds = &g.devices[q->dev];
  std::lock_guard<std::mutex> lock(ds->mu);
  ds->free_blocks.push_back(QueueBlock{q->meta, q->meta_dev, q->dev_handle, q->stage, q->stage_dev});
  delete q;
}

void unpack_queue_next_free(UnpackQueue* q, UnpackSlot* slot) {
  if (q->tail - q->head >= static_cast<uint64_t>(kQueueDepth)) {
    *slot = UnpackSlot{};  // inactive, all pointers null
    return;
  }
  const uint64_t idx = q->tail % kQueueDepth;
  slot->active = true;
  slot->idx = idx;
  slot->mem = q->meta->nccl.mem[idx];
  slot->cnt = &q->meta->nccl.cnt[idx];
  slot->cnt_cache = 0;
  slot->flow_cnt = &q->record.flow_cnts[idx];
  slot->pgtok_cnts = q->record.pgtok_cnts[idx];
  slot->flows = q->record.flows[idx];
  slot->pgtoks = &q->record.pgtoks[idx][0][0];
  q->tail += 1;
}

}  // namespace tcpx
