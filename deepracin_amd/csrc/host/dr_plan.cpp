// Graph core: execution order, buffer planning, weight upload, teardown.
//
// Execution order follows the reference's work-list walk (src/dR_core.c:121-211): a FIFO seeded
// with the consumers of the feed nodes in feed order; a node whose producers are not all done goes
// to the back of the queue; a finished node appends its not-yet-queued consumers.  The order in
// which nodes finish is the schedule.
//
// Buffer planning differs from the reference on purpose.  The reference recycles "stream buffers"
// with a reference count while it walks the schedule (src/dR_core.c:213-325).  Here every tensor
// gets a live interval [first writer, last reader] in schedule positions and physical buffers are
// assigned by interval; on top of that a channel Concat whose inputs are produced for it alone is
// planned as ONE buffer into which the producers write at their channel offset, so the concat
// itself moves no data.  Externally visible guarantees are the reference's: feed buffers and
// buffers of output nodes are never recycled, and a node never writes the buffer it reads.
#include "dr_internal.hpp"

#include <algorithm>
#include <deque>
#include <map>

using namespace dr;

namespace {

// A tensor that owns storage (a "root"): either a plain node output or a fused concat buffer
// together with all the producer outputs that live inside it.
struct Root {
    dR_Node* owner = nullptr;
    int size = 0;             // floats
    int firstDef = 1 << 30;   // schedule position of the earliest writer
    int lastUse = -1;         // schedule position of the latest reader
    bool pinned = false;      // feed/output/caller-supplied: never shares storage
    dR_MemoryHandler* phys = nullptr;
};

// A node whose tensor has to exist in memory after the pass although the graph has one reader for it: an output
// node, or the layer the caller asked a debug download of (dR_Graph::debugLayer, read when the buffers are planned).
thread_local int g_debugLayerAtPlanTime = -1;
inline bool tensor_wanted(const dR_Node* n) { return n->output || n->layerID == g_debugLayerAtPlanTime; }

bool concat_can_fuse(const dR_Node* c) {
    if (c->type != tConcat) return false;
    const dR_Concat_Data* cd = (const dR_Concat_Data*)c->layer;
    if (cd->concatDim != 2) return false;
    if (c->outputBuf && c->outputBuf->outputBuf) return false;  // caller-supplied storage
    std::vector<dR_Node*> ins = nodes_of(c->previous_layers);
    int off = 0;    // floats in front of producer i inside the joint buffer
    for (size_t i = 0; i < ins.size(); ++i) {
        const dR_Node* p = ins[i];
        // The normalization kernels move 16 bytes per lane and refuse other addresses: such a producer
        // may only sit at a multiple of 4 floats (buffers themselves start 256-byte aligned).
        if (p->type == tNormalization && (off & 3)) return false;
        off += p->oshape.s0 * p->oshape.s1 * p->oshape.s2;
        if (p->type == tDataFeedNode || tensor_wanted(p)) return false;
        if (!p->next_layers || p->next_layers->length != 1) return false;
        if (p->outputBuf) return false;     // already bound to a caller buffer
        if (p->oshape.s0 != c->oshape.s0 || p->oshape.s1 != c->oshape.s1) return false;
        for (size_t j = 0; j < i; ++j) if (ins[j] == p) return false;
    }
    return !ins.empty();
}

// The expand pair of a fire module: a 1x1 and a 3x3 convolution of the same tensor whose outputs sit
// next to each other in a fused channel concat.  A 1x1 filter is a 3x3 filter with only its centre
// tap, so both become ONE Winograd launch over the joint output channels (DR_FUSE_EXPAND=0 keeps
// them apart).  The 1x1 outputs then come out of the Winograd transforms instead of the plain
// dot product: same function, fp32 rounding differs at the 1e-6 level.
bool expand_pair(const dR_Node* a, const dR_Node* b) {
    const char* env = getenv("DR_FUSE_EXPAND");
    if (env && strcmp(env, "0") == 0) return false;
    if (a->type != tConv2d || b->type != tConv2d) return false;
    const dR_Conv2d_Data* ca = (const dR_Conv2d_Data*)a->layer;
    const dR_Conv2d_Data* cb = (const dR_Conv2d_Data*)b->layer;
    if (ca->algo != drConv1x1Gemm || cb->algo != drConvWinograd) return false;
    if (ca->activation != cb->activation || ca->shape.s2 != cb->shape.s2) return false;
    std::vector<dR_Node*> ia = nodes_of(a->previous_layers), ib = nodes_of(b->previous_layers);
    return ia.size() == 1 && ib.size() == 1 && ia[0] == ib[0];
}

// Max pooling stored by the convolution in front of it, so that the full-resolution tensor never
// exists (only when nobody else wants that tensor; DR_FUSE_POOL=0 keeps the two apart):
//  - a 2x2 / stride-2 pool behind a Winograd convolution: every 2x2 output tile of the convolution
//    is one pooling window;
//  - a 3x3 / stride-2 pool behind a first layer (3x3 filter, at most 4 input channels): one kernel
//    computes the convolution outputs of a pooled tile on the matrix cores and pools them in LDS.
dR_Node* pool_fusable_producer(const dR_Node* p) {
    if (p->type != tPooling) return nullptr;
    const char* env = getenv("DR_FUSE_POOL");
    if (env && strcmp(env, "0") == 0) return nullptr;
    const dR_Pooling_Data* pd = (const dR_Pooling_Data*)p->layer;
    if (pd->poolingType != tMax || pd->shape.s3 != 1 || pd->stride.s1 != 2 || pd->stride.s2 != 2 || pd->stride.s3 != 1) return nullptr;
    const bool two = pd->shape.s1 == 2 && pd->shape.s2 == 2, three = pd->shape.s1 == 3 && pd->shape.s2 == 3;
    if (!two && !three) return nullptr;
    std::vector<dR_Node*> ins = nodes_of(p->previous_layers);
    if (ins.size() != 1) return nullptr;
    dR_Node* c = ins[0];
    if (c->type != tConv2d) return nullptr;
    const dR_Conv2d_Data* cd = (const dR_Conv2d_Data*)c->layer;
    if (tensor_wanted(c) || c->outputBuf || !c->next_layers || c->next_layers->length != 1) return nullptr;
    if (two) {
        if (cd->algo != drConvWinograd || ((c->oshape.s0 | c->oshape.s1) & 1)) return nullptr;
    } else {
        if (cd->algo != drConvDirect || cd->shape.s0 != 3 || cd->shape.s1 != 3 || cd->shape.s2 > 4) return nullptr;
        // (that kernel carries its shape in 16-bit fields and its strides in 4-bit fields)
        if (cd->ishape.s0 > 65535 || cd->ishape.s1 > 65535 || cd->shape.s3 > 65535 || cd->stride.s1 > 15 || cd->stride.s2 > 15) return nullptr;
    }
    return c;
}

// A 3x3 / stride-2 max pooling whose only reader is a 1x1 convolution: the convolution takes the window maxima
// while it loads its input, the pooled tensor is never written and the pooling kernel is not launched
// (DR_FUSE_POOLIN=0 keeps them apart).  Returns the pooling node in front of such a convolution.
dR_Node* pooled_input_of(const dR_Node* c) {
    if (c->type != tConv2d) return nullptr;
    const char* env = getenv("DR_FUSE_POOLIN");
    if (env && strcmp(env, "0") == 0) return nullptr;
    const dR_Conv2d_Data* cd = (const dR_Conv2d_Data*)c->layer;
    if (cd->algo != drConv1x1Gemm) return nullptr;
    std::vector<dR_Node*> ins = nodes_of(c->previous_layers);
    if (ins.size() != 1 || ins[0]->type != tPooling) return nullptr;
    dR_Node* p = ins[0];
    const dR_Pooling_Data* pd = (const dR_Pooling_Data*)p->layer;
    if (pd->poolingType != tMax || pd->shape.s1 != 3 || pd->shape.s2 != 3 || pd->shape.s3 != 1) return nullptr;
    if (pd->stride.s1 != 2 || pd->stride.s2 != 2 || pd->stride.s3 != 1) return nullptr;
    if (tensor_wanted(p) || p->outputBuf || !p->next_layers || p->next_layers->length != 1) return nullptr;
    if (pool_fusable_producer(p)) return nullptr;      // already stored by the convolution in front of it
    // (the pooling-on-load kernel addresses the unpooled tensor with 32-bit byte offsets)
    if ((long long)pd->ishape.s0 * pd->ishape.s1 * pd->ishape.s2 >= (1ll << 29)) return nullptr;
    return p;
}

// A global average pooling (one window = the whole map) behind a 1x1 convolution and in front of an
// FC or softmax node: the convolution's epilogue sums its pixels per tile, the consumer adds the
// tile sums and divides, and neither the convolution's tensor nor a pooling kernel is needed
// (DR_FUSE_AVGPOOL=0 keeps them).  The pooled tensor may still be an output: the consumer stores it.
dR_Node* avgpool_fusable_producer(const dR_Node* p) {
    if (p->type != tPooling) return nullptr;
    const char* env = getenv("DR_FUSE_AVGPOOL");
    if (env && strcmp(env, "0") == 0) return nullptr;
    const dR_Pooling_Data* pd = (const dR_Pooling_Data*)p->layer;
    if (pd->poolingType != tAverage || pd->shape.s3 != 1 || pd->stride.s3 != 1) return nullptr;
    if (pd->shape.s1 != pd->ishape.s0 || pd->shape.s2 != pd->ishape.s1) return nullptr;
    if (pd->stride.s1 < pd->ishape.s0 || pd->stride.s2 < pd->ishape.s1) return nullptr;
    if (p->outputBuf || !p->next_layers || p->next_layers->length != 1) return nullptr;
    const dR_Node* consumer = nodes_of(p->next_layers)[0];
    if (consumer->type != tFullyConnected && consumer->type != tSoftmax) return nullptr;
    std::vector<dR_Node*> ins = nodes_of(p->previous_layers);
    if (ins.size() != 1) return nullptr;
    dR_Node* c = ins[0];
    if (c->type != tConv2d || ((const dR_Conv2d_Data*)c->layer)->algo != drConv1x1Gemm) return nullptr;
    if (tensor_wanted(c) || c->outputBuf || !c->next_layers || c->next_layers->length != 1) return nullptr;
    return c;
}

}  // namespace

extern "C" {

dR_Graph* dR_appendLayer(dR_Graph* net, dR_Node* l) {
    l->propagated = FALSE;
    l->output = FALSE;
    l->queued = FALSE;
    l->layerID = net->number_of_layers;
    l->drSchedulePos = -1;
    l->drLastKernelMs = 0.f;
    if (l->type != tDataFeedNode) l->outputBuf = NULL;
    dR_list_append(net->allNodes, l);
    net->number_of_layers++;
    return net;
}

gboolean dR_propagateShapesAndSchedule(dR_Graph* net) {
    if (net->feed_layers->length == 0) {
        say("A minimum of one data feed node is required to prepare the net application!\n");
        return FALSE;
    }
    std::deque<dR_Node*> work;
    auto enqueue_consumers = [&](dR_Node* n) {
        for_each(n->next_layers, [&](void* p) {
            dR_Node* c = (dR_Node*)p;
            if (!c->queued) { c->queued = TRUE; work.push_back(c); }
        });
    };
    for (dR_Node* feed : nodes_of(net->feed_layers)) {
        feed->oshape = ((dR_DataFeedNode_Data*)feed->layer)->shape;
        feed->propagated = TRUE;
        enqueue_consumers(feed);
    }

    dR_List* order = dR_list_createEmptyList();
    size_t stalled = 0;     // consecutive deferrals; == work.size() means nobody can make progress
    int pos = 0;
    while (!work.empty()) {
        dR_Node* n = work.front();
        work.pop_front();
        bool ready = true;
        for_each(n->previous_layers, [&](void* p) { ready = ready && ((dR_Node*)p)->propagated; });
        if (!ready) {
            work.push_back(n);
            if (++stalled > work.size()) {
                say("Scheduling failed: node %d depends on a node no feed node reaches.\n", n->layerID);
                dR_list_cleanup(order);
                return FALSE;
            }
            continue;
        }
        stalled = 0;
        if (!n->propagateShape(net, n)) {
            say("Propagate Shapes failed for Layer %d!", n->layerID);
            dR_list_cleanup(order);
            return FALSE;
        }
        if (debug(net)) say("Propagated layer %d: %dx%dx%d\n", n->layerID, n->oshape.s0, n->oshape.s1, n->oshape.s2);
        if (!n->schedule(net, n)) {
            say("Scheduling failed for Layer %d! \n", n->layerID);
            dR_list_cleanup(order);
            return FALSE;
        }
        n->propagated = TRUE;
        n->drSchedulePos = pos++;
        dR_list_append(order, n);
        enqueue_consumers(n);
    }
    net->scheduledLayers = order;
    if (debug(net)) dR_printSchedule(net);
    return TRUE;
}

// Kernels are compiled ahead of time; what is left of this stage is the per-node hook.
gboolean dR_generateAndCompileKernels(dR_Graph* net) {
    for (dR_Node* n : nodes_of(net->scheduledLayers)) {
        if (n->generateKernel && !n->generateKernel(net, n)) {
            say("Kernel Generation failed for Layer %d! \n", n->layerID);
            return FALSE;
        }
        if (n->createKernel && !n->createKernel(net, n)) {
            say("Kernel selection failed for Layer %d! \n", n->layerID);
            return FALSE;
        }
    }
    return TRUE;
}

dR_MemoryHandler* dR_newMemoryHandler(gboolean custom) {
    dR_MemoryHandler* h = zalloc<dR_MemoryHandler>();
    h->outputFor = dR_list_createEmptyList();
    h->outputBuf = custom;
    h->bufptr = &h->buf;
    h->drFirstDef = 1 << 30;
    h->drLastUse = -1;
    return h;
}

void dR_cleanupMemoryHandler(dR_Graph* net, dR_MemoryHandler* h) {
    if (!h) return;
    if (!h->outputBuf && !h->drViewOf) dR_clMemoryBufferCleanup(net, h->buf);
    dR_list_cleanup(h->outputFor);
    free(h);
}

gboolean dR_planBuffers(dR_Graph* net) {
    if (!net->scheduledLayers) { say("dR_planBuffers: graph has no schedule yet\n"); return FALSE; }
    std::vector<dR_Node*> sched = nodes_of(net->scheduledLayers);
    std::vector<dR_Node*> feeds = nodes_of(net->feed_layers);
    g_debugLayerAtPlanTime = net->debugLayer;

    // 1. which concat nodes absorb their producers
    std::map<dR_Node*, std::pair<dR_Node*, int>> parent;   // producer -> (concat, float offset)
    // FC -> FC and FC -> softmax: the consumer sums the producer's split-K partials while it loads
    // its input, the producer's finishing kernel is not launched (DR_FUSE_FC=0 keeps it).
    for (dR_Node* n : sched) {
        if (n->type == tFullyConnected) { ((dR_FC_Data*)n->layer)->drDeferReduce = FALSE; ((dR_FC_Data*)n->layer)->drDeferredInput = nullptr; }
        if (n->type == tSoftmax) ((dR_Softmax_Data*)n->layer)->drDeferredInput = nullptr;
    }
    const char* fuseFc = getenv("DR_FUSE_FC");
    for (dR_Node* n : sched) {
        if (n->type != tFullyConnected || (fuseFc && strcmp(fuseFc, "0") == 0)) continue;
        dR_FC_Data* fd = (dR_FC_Data*)n->layer;
        // an output node can defer too: its consumer stores the finished vector into its buffer
        if (n->outputBuf || !n->next_layers || n->next_layers->length != 1 || n->layerID == g_debugLayerAtPlanTime) continue;
        if (drhip_fc_slices(fd->shape.s0, fd->shape.s1) <= 1) continue;
        dR_Node* c = nodes_of(n->next_layers)[0];
        if (c->type == tFullyConnected) ((dR_FC_Data*)c->layer)->drDeferredInput = n;
        else if (c->type == tSoftmax) ((dR_Softmax_Data*)c->layer)->drDeferredInput = n;
        else continue;
        fd->drDeferReduce = TRUE;
    }
    for (dR_Node* n : sched)
        if (n->type == tConv2d) ((dR_Conv2d_Data*)n->layer)->drAbsorbed1x1 = ((dR_Conv2d_Data*)n->layer)->drAbsorbedBy = nullptr;
    for (dR_Node* n : sched)
        if (n->type == tConv2d) ((dR_Conv2d_Data*)n->layer)->drFusedPool = ((dR_Conv2d_Data*)n->layer)->drFusedAvgPool = FALSE;
    for (dR_Node* n : sched)
        if (n->type == tConv2d) ((dR_Conv2d_Data*)n->layer)->drPooledInput = nullptr;
    for (dR_Node* n : sched) {
        if (n->type == tPooling) {
            dR_Node* c = pool_fusable_producer(n);
            ((dR_Pooling_Data*)n->layer)->drFused = c != nullptr;
            if (c) { ((dR_Conv2d_Data*)c->layer)->drFusedPool = TRUE; parent[c] = std::make_pair(n, 0); }
            else if ((c = avgpool_fusable_producer(n)) != nullptr) {
                dR_Node* consumer = nodes_of(n->next_layers)[0];
                if (consumer->type == tFullyConnected) ((dR_FC_Data*)consumer->layer)->drDeferredInput = n;
                else ((dR_Softmax_Data*)consumer->layer)->drDeferredInput = n;
                ((dR_Conv2d_Data*)c->layer)->drFusedAvgPool = TRUE;
                ((dR_Pooling_Data*)n->layer)->drFused = TRUE;
            }
        }
        if (n->type != tConcat) continue;
        dR_Concat_Data* cd = (dR_Concat_Data*)n->layer;
        cd->drFused = concat_can_fuse(n);
        if (!cd->drFused) continue;
        int off = 0;
        std::vector<dR_Node*> ins = nodes_of(n->previous_layers);
        for (dR_Node* p : ins) {
            parent[p] = std::make_pair(n, off);
            off += p->oshape.s0 * p->oshape.s1 * p->oshape.s2;
        }
        for (size_t k = 0; k + 1 < ins.size(); ++k)
            if (expand_pair(ins[k], ins[k + 1]) && !((dR_Conv2d_Data*)ins[k]->layer)->drAbsorbedBy) {
                ((dR_Conv2d_Data*)ins[k]->layer)->drAbsorbedBy = ins[k + 1];
                ((dR_Conv2d_Data*)ins[k + 1]->layer)->drAbsorbed1x1 = ins[k];
            }
    }
    // (after the loop above: whether a 1x1 layer feeds a fused global average is known only now)
    for (dR_Node* n : sched) {
        if (n->type != tConv2d || ((dR_Conv2d_Data*)n->layer)->drFusedAvgPool) continue;
        if (dR_Node* pool = pooled_input_of(n)) {
            ((dR_Conv2d_Data*)n->layer)->drPooledInput = pool;
            ((dR_Pooling_Data*)pool->layer)->drFused = TRUE;
        }
    }
    auto root_of = [&](dR_Node* n, int* offset) {
        int off = 0;
        std::map<dR_Node*, std::pair<dR_Node*, int>>::iterator it;
        while ((it = parent.find(n)) != parent.end()) { off += it->second.second; n = it->second.first; }
        if (offset) *offset = off;
        return n;
    };

    // 2. live interval per root
    std::map<dR_Node*, Root> roots;
    std::vector<dR_Node*> rootOrder;
    auto touch = [&](dR_Node* owner) -> Root& {
        std::map<dR_Node*, Root>::iterator it = roots.find(owner);
        if (it == roots.end()) {
            Root r;
            r.owner = owner;
            r.size = owner->getRequiredOutputBufferSize(owner);
            r.pinned = owner->type == tDataFeedNode || owner->output || (owner->outputBuf && owner->outputBuf->outputBuf);
            it = roots.insert(std::make_pair(owner, r)).first;
            rootOrder.push_back(owner);
        }
        return it->second;
    };
    for (dR_Node* f : feeds) { Root& r = touch(f); r.firstDef = -1; }
    for (dR_Node* n : sched) {
        Root& r = touch(root_of(n, nullptr));
        r.firstDef = std::min(r.firstDef, n->drSchedulePos);
        r.lastUse = std::max(r.lastUse, n->drSchedulePos);
        for (dR_Node* p : nodes_of(n->previous_layers)) {
            Root& rp = touch(root_of(p, nullptr));
            rp.lastUse = std::max(rp.lastUse, n->drSchedulePos);
        }
        // a convolution that pools while loading reads the tensor in front of the pooling node
        if (n->type == tConv2d && ((dR_Conv2d_Data*)n->layer)->drPooledInput) {
            for (dR_Node* p : nodes_of(((dR_Conv2d_Data*)n->layer)->drPooledInput->previous_layers)) {
                Root& rp = touch(root_of(p, nullptr));
                rp.lastUse = std::max(rp.lastUse, n->drSchedulePos);
            }
        }
    }

    // 3. assign physical buffers in order of first definition; best fit among the free ones
    dR_List* handlers = dR_list_createEmptyList();
    std::vector<dR_MemoryHandler*> pool;    // recyclable physical buffers
    std::stable_sort(rootOrder.begin(), rootOrder.end(),
                     [&](dR_Node* a, dR_Node* b) { return roots[a].firstDef < roots[b].firstDef; });
    for (dR_Node* owner : rootOrder) {
        Root& r = roots[owner];
        dR_MemoryHandler* h = nullptr;
        if (owner->outputBuf && owner->outputBuf->outputBuf) {
            h = owner->outputBuf;               // caller-supplied: keep as is
            h->drPinned = TRUE;
        } else if (r.pinned) {
            h = dR_newMemoryHandler(FALSE);
            h->drPinned = TRUE;
            dR_list_append(handlers, h);
        } else {
            int best = -1;
            for (size_t i = 0; i < pool.size(); ++i) {
                if (pool[i]->drLastUse >= r.firstDef) continue;          // still being read
                if (best < 0) { best = (int)i; continue; }
                const int sb = pool[best]->size, si = pool[i]->size;
                const bool fitb = sb >= r.size, fiti = si >= r.size;
                if ((fiti && !fitb) || (fiti && fitb && si < sb) || (!fiti && !fitb && si > sb)) best = (int)i;
            }
            if (best >= 0) h = pool[best];
            else { h = dR_newMemoryHandler(FALSE); pool.push_back(h); dR_list_append(handlers, h); }
        }
        h->size = std::max(h->size, r.size);
        h->drFirstDef = std::min(h->drFirstDef, r.firstDef);
        h->drLastUse = std::max(h->drLastUse, r.lastUse);
        r.phys = h;
    }

    // 4. bind nodes: roots get the physical handler, absorbed producers get a view into it
    auto bind = [&](dR_Node* n) {
        int off = 0;
        dR_Node* owner = root_of(n, &off);
        dR_MemoryHandler* phys = roots[owner].phys;
        if (owner == n) {
            n->outputBuf = phys;
            phys->numberOfDependencies = n->next_layers ? n->next_layers->length : 0;
            dR_list_append(phys->outputFor, n);
        } else {
            dR_MemoryHandler* v = dR_newMemoryHandler(FALSE);
            v->drViewOf = phys;
            v->drViewOffset = off;
            v->size = n->getRequiredOutputBufferSize(n);
            v->numberOfDependencies = 1;
            dR_list_append(v->outputFor, n);
            dR_list_append(net->drViewHandlers, v);
            n->outputBuf = v;
        }
    };
    for (dR_Node* f : feeds) bind(f);
    for (dR_Node* n : sched) bind(n);

    net->streamBufferHandlers = handlers;
    int maxSize = 0;
    for_each(handlers, [&](void* p) { maxSize = std::max(maxSize, ((dR_MemoryHandler*)p)->size); });
    net->maxBufferSize = maxSize;
    if (debug(net)) say("Number of required stream buffers: %d\n", handlers->length);
    return TRUE;
}

gboolean dR_estimateAndAllocateBuffers(dR_Graph* net) {
    if (!dR_planBuffers(net)) return FALSE;
    gboolean ok = TRUE;
    for_each(net->streamBufferHandlers, [&](void* p) {
        dR_MemoryHandler* h = (dR_MemoryHandler*)p;
        h->bufptr = &h->buf;
        ok = ok && dR_createFloatBuffer(net, h->bufptr, h->size, CL_MEM_READ_WRITE);
        if (debug(net)) say("Stream buffer with size %d created!\n", h->size);
    });
    if (!ok) return FALSE;
    for_each(net->drViewHandlers, [&](void* p) {
        dR_MemoryHandler* v = (dR_MemoryHandler*)p;
        v->buf = (cl_mem)((float*)v->drViewOf->buf + v->drViewOffset);
        v->bufptr = &v->buf;
    });
    // per-node parameter buffers (weights, biases, scratch)
    for (dR_Node* f : nodes_of(net->feed_layers))
        if (f->allocateBuffers && !f->allocateBuffers(net, f)) { say("Buffer allocation failed for Layer %d! \n", f->layerID); return FALSE; }
    for (dR_Node* n : nodes_of(net->scheduledLayers))
        if (!n->allocateBuffers(net, n)) { say("Buffer allocation failed for Layer %d! \n", n->layerID); return FALSE; }
    net->hostDebugBuffer = (cl_float*)malloc((size_t)std::max(net->maxBufferSize, 1) * sizeof(float));
    return TRUE;
}

gboolean dR_fillBuffers(dR_Graph* net) {
    for (dR_Node* n : nodes_of(net->scheduledLayers))
        if (!n->fillBuffers(net, n)) { say("Buffer filling failed for Layer %d! \n", n->layerID); return FALSE; }
    return TRUE;
}

void dR_cleanupBuffers(dR_Graph* net) {
    for_each(net->streamBufferHandlers, [&](void* p) {
        dR_MemoryHandler* h = (dR_MemoryHandler*)p;
        if (!dR_clMemoryBufferCleanup(net, h->buf)) say("Stream buffer cleanup failed \n");
        h->buf = NULL;
    });
    for (dR_Node* n : nodes_of(net->scheduledLayers))
        if (n->cleanupBuffers && !n->cleanupBuffers(net, n)) say("Buffer cleanup failed for Layer %d! \n", n->layerID);
}

void dR_cleanupNet(dR_Graph* net) {
    auto drop_handlers = [&](dR_List* l) {
        for_each(l, [&](void* p) { dR_MemoryHandler* h = (dR_MemoryHandler*)p; dR_list_cleanup(h->outputFor); free(h); });
        dR_list_cleanup(l);
    };
    if (net->streamBufferHandlers) drop_handlers(net->streamBufferHandlers);
    drop_handlers(net->drViewHandlers);
    for (dR_Node* n : nodes_of(net->allNodes)) {
        if (n->cleanupLayer && !n->cleanupLayer(net, n)) say("Layer cleanup failed for layer %d! \n", n->layerID);
        dR_list_cleanup(n->previous_layers);
        dR_list_cleanup(n->next_layers);
        free(n);
    }
    if (net->scheduledLayers) dR_list_cleanup(net->scheduledLayers);
    free(net->hostDebugBuffer);
    dR_list_cleanup(net->allNodes);
    dR_list_cleanup(net->output_layers);
    dR_list_cleanup(net->feed_layers);
    free(net->clConfig);
    free(net->config);
    free(net);
}

// ---- data feed node (reference src/dR_core.c:18-119) ----------------------------------------------

static gchar* feed_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_DataFeedNode_Data* d = (dR_DataFeedNode_Data*)node->layer;
    if (*numParams < 3) { say("DataFeedNode needs space for 3 parameters and 0 variables!\n"); return NULL; }
    *numParams = 3;
    params[0] = fmt_dup("%d", d->shape.s0);
    params[1] = fmt_dup("%d", d->shape.s1);
    params[2] = fmt_dup("%d", d->shape.s2);
    *numVariables = 0;
    return (gchar*)"DataFeedNode";
}

static gchar* feed_print(dR_Node* node) {
    dR_DataFeedNode_Data* d = (dR_DataFeedNode_Data*)node->layer;
    return fmt_dup("DataFeedNode: %d\n Data dimensions: %dx%dx%d\n", node->layerID, d->shape.s0, d->shape.s1, d->shape.s2);
}

static gint32 feed_size(dR_Node* node) {
    dR_DataFeedNode_Data* d = (dR_DataFeedNode_Data*)node->layer;
    return d->shape.s0 * d->shape.s1 * d->shape.s2;
}

static gboolean feed_noop(dR_Graph*, dR_Node*) { return TRUE; }
static gboolean feed_cleanup(dR_Graph*, dR_Node* node) { free(node->layer); node->layer = NULL; return TRUE; }

dR_Node* dR_datafeednode_parseAppendNode(dR_Graph* net, dR_Node**, gint numINodes, gchar** params, gint numParams,
                                         gfloat**, gint numVariables) {
    if (numINodes != 0) { say("Parsing Error: DataFeedNode Node needs 0 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 3 || numVariables != 0) { say("Parsing Error: DataFeedNode Node needs 3 Parameters and 0 Variables!\n"); return NULL; }
    dR_Shape3 s = { atoi(params[0]), atoi(params[1]), atoi(params[2]) };
    return dR_Datafeednode(net, &s);
}

dR_Node* dR_Datafeednode(dR_Graph* net, dR_Shape3* shape) {
    dR_DataFeedNode_Data* d = zalloc<dR_DataFeedNode_Data>();
    dR_Node* n = zalloc<dR_Node>();
    d->shape = *shape;
    n->layer = d;
    n->type = tDataFeedNode;
    n->next_layers = dR_list_createEmptyList();
    n->previous_layers = dR_list_createEmptyList();
    n->printLayer = feed_print;
    n->allocateBuffers = feed_noop;     // storage comes from the buffer planner
    n->fillBuffers = feed_noop;
    n->cleanupBuffers = feed_noop;
    n->getRequiredOutputBufferSize = feed_size;
    n->cleanupLayer = feed_cleanup;
    n->serializeNode = feed_serialize;
    n->parseAppendNode = dR_datafeednode_parseAppendNode;
    dR_list_append(net->feed_layers, n);
    dR_appendLayer(net, n);
    return n;
}

}  // extern "C"
