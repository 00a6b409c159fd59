/*
 * flow_mapper.h -- which data flow takes the next chunk of a message.
 *
 * The reference keeps one scheduler per comm (class FlowMapper, src/flow_mapper.h:52-65), refills it at every
 * progress call with the flows whose task ring has room (src/net_tcpx.cc:1114,1152-1155), proceeds only if it
 * holds a flow (src/net_tcpx.cc:1183), and -- on the sending side -- asks it which flow the next chunk goes to
 * (src/net_tcpx.cc:1216).  Two policies, chosen by NCCL_GPUDIRECTTCPX_SCHED_ALG (src/net_tcpx.cc:643-665):
 *   RR    the flows with room, handed out last scheduled first           (FlowMapperRR,   src/flow_mapper.h:137-157)
 *   KATY  the flow with the most free task slots first, at most two      (FlowMapperKaty, src/flow_mapper.h:67-135)
 *         chunks per progress call; a flow that was picked stays scheduled one priority lower
 * The receive path uses reset / schedule / has_flow; pick is what a sender (here: the synthetic peer) calls.
 */
#ifndef TCPX_AMD_FLOW_MAPPER_H_
#define TCPX_AMD_FLOW_MAPPER_H_

#include <stdint.h>
#include <strings.h>

namespace tcpx {

constexpr int kSchedRoundRobin = 0;  // TCPX_FLOWMAPPER_SCHED_ALG_RR (default)
constexpr int kSchedKaty = 1;        // TCPX_FLOWMAPPER_SCHED_ALG_KATY

class FlowScheduler {
 public:
  virtual ~FlowScheduler() = default;
  virtual void reset() = 0;
  virtual bool has_flow() const = 0;
  // prio = task slots in use on the flow, 0 (idle, served first) .. max_tasks - 1.
  virtual void schedule(int flow, int prio) = 0;
  virtual int pick() = 0;  // a flow, or -1
};

class RoundRobinFlows final : public FlowScheduler {
 public:
  void reset() override { n_ = 0; }
  bool has_flow() const override { return n_ > 0; }
  void schedule(int flow, int /*prio*/) override {
    if (n_ < kCapacity) flows_[n_++] = flow;
  }
  int pick() override { return n_ > 0 ? flows_[--n_] : -1; }

 private:
  static constexpr int kCapacity = 8;  // MAX_SOCKETS
  int flows_[kCapacity];
  int n_ = 0;
};

class KatyFlows final : public FlowScheduler {
 public:
  KatyFlows(int max_flows, int max_tasks) : max_flows_(max_flows), max_tasks_(max_tasks) {}
  void reset() override {
    bitmap_ = 0;
    quanta_ = kQuantaPerRound;
  }
  bool has_flow() const override { return bitmap_ != 0 && quanta_ > 0; }
  void schedule(int flow, int prio) override {
    if (prio < 0 || prio >= max_tasks_ || flow < 0 || flow >= max_flows_) return;
    bitmap_ |= 1ull << (flow + max_flows_ * prio);  // bit = flow within the group of its priority
  }
  int pick() override {
    if (!has_flow()) return -1;
    const int bit = ffsll(static_cast<long long>(bitmap_)) - 1;  // lowest bit: highest priority, lowest flow
    const int prio = bit / max_flows_, flow = bit % max_flows_;
    bitmap_ &= ~(1ull << bit);
    if (prio < max_tasks_ - 1) bitmap_ |= 1ull << (bit + max_flows_);  // still has room: one priority lower
    --quanta_;
    return flow;
  }

 private:
  static constexpr int kQuantaPerRound = 2;  // NUM_QUANTA_PER_SCHED
  const int max_flows_, max_tasks_;
  uint64_t bitmap_ = 0;
  int quanta_ = kQuantaPerRound;
};

}  // namespace tcpx

#endif  // TCPX_AMD_FLOW_MAPPER_H_
