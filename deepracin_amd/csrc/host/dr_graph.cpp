// Graph life cycle of the deepRacin C API on top of the HIP device layer:
// dR_NewGraph / dR_config / dR_initCL / dR_prepare / dR_apply / dR_feedData / dR_getOutputBuffers /
// dR_downloadArray / dR_cleanup.  Same call contract as the reference's src/deepRACIN.c and the
// buffer helpers of src/dR_clwrap.c; everything underneath is HIP.
#include "dr_internal.hpp"

#include <algorithm>
#include <chrono>
#include <vector>

using namespace dr;

// ---- recording the forward pass into a stream capture ------------------------------------------
//
// Nodes are recorded in schedule order on the graph's stream.  Consecutive nodes that do not depend
// on each other (the two expand convolutions of a fire module) are recorded on side streams between
// a fork and a join event when DR_BRANCHES=1 is set, so the captured graph runs them concurrently.
// Off by default: on MI355X with ROCm 7.2 every fork/join edge of a replayed graph costs more
// (SqueezeNet v1.1: 0.226 ms per pass with the 8 expand pairs forked, 0.211 ms in one chain) than
// the overlap of two ~8 us kernels returns.  The buffer plan assumes schedule order, so a group
// is only formed when no member writes memory another member reads or writes.

struct Range { const char* lo; const char* hi; };

static Range out_range(dR_Node* n) {
    const char* p = (const char*)dev_out(n);
    return Range{p, p + (size_t)n->oshape.s0 * n->oshape.s1 * n->oshape.s2 * sizeof(float)};
}
static bool overlap(const Range& a, const Range& b) { return a.lo && b.lo && a.lo < b.hi && b.lo < a.hi; }

static bool can_run_beside(dR_Node* a, dR_Node* b) {
    for (dR_Node* p : nodes_of(b->previous_layers)) if (p == a) return false;
    for (dR_Node* p : nodes_of(a->previous_layers)) if (p == b) return false;
    const Range wa = out_range(a), wb = out_range(b);
    if (overlap(wa, wb)) return false;
    for (dR_Node* p : nodes_of(a->previous_layers)) if (overlap(out_range(p), wb)) return false;
    for (dR_Node* p : nodes_of(b->previous_layers)) if (overlap(out_range(p), wa)) return false;
    return true;
}

static bool record_forward_pass(dR_Graph* net) {
    dR_ClConfig* cc = net->clConfig;
    void* const mainStream = cc->hipStream;
    const char* env = getenv("DR_BRANCHES");
    bool branches = env && strcmp(env, "1") == 0;
    if (branches && !net->drBranchEvents[0]) {
        for (int k = 0; k < 3 && branches; ++k) branches = drhip_stream_create(&net->drSideStreams[k]) == DRHIP_OK;
        for (int k = 0; k < 4 && branches; ++k) branches = drhip_event_create(&net->drBranchEvents[k]) == DRHIP_OK;
    }
    std::vector<dR_Node*> sched = nodes_of(net->scheduledLayers);
    net->drBranchGroups = 0;
    bool ok = true;
    for (size_t i = 0; i < sched.size() && ok;) {
        size_t j = i + 1;
        while (branches && j < sched.size() && j - i < 4) {
            bool free = sched[j]->type != tConcat;
            for (size_t m = i; m < j && free; ++m) free = sched[m]->type != tConcat && can_run_beside(sched[m], sched[j]);
            if (!free) break;
            ++j;
        }
        if (j - i == 1) {
            ok = sched[i]->compute(net, sched[i]);
        } else {
            ok = drhip_event_record(net->drBranchEvents[0], mainStream) == DRHIP_OK;
            for (size_t m = i + 1; m < j && ok; ++m) {
                void* side = net->drSideStreams[m - i - 1];
                ok = drhip_stream_wait_event(side, net->drBranchEvents[0]) == DRHIP_OK;
                cc->hipStream = side;                // the node launches on whatever the graph's stream is
                ok = ok && sched[m]->compute(net, sched[m]);
                cc->hipStream = mainStream;
                ok = ok && drhip_event_record(net->drBranchEvents[m - i], side) == DRHIP_OK;
            }
            ok = ok && sched[i]->compute(net, sched[i]);
            for (size_t m = i + 1; m < j; ++m)       // join even after a failure: the capture must end on one stream
                ok = (drhip_stream_wait_event(mainStream, net->drBranchEvents[m - i]) == DRHIP_OK) && ok;
            net->drBranchGroups++;
        }
        i = j;
    }
    return ok;
}

extern "C" {

// Defaults as in the reference (src/deepRACIN.c:6-47): silent, no profiling, first GPU.
dR_Graph* dR_NewGraph(void) {
    dR_Graph* g = zalloc<dR_Graph>();
    g->clConfig = zalloc<dR_ClConfig>();
    g->config = zalloc<dR_Config>();

    dR_ClConfig* cc = g->clConfig;
    cc->clEvent = &cc->clEventObject;
    cc->clDeviceType = CL_DEVICE_TYPE_GPU;
    cc->clDeviceNumber = 0;
    cc->clInfo = TRUE;
    cc->clKernelPath = (gchar*)"";
    cc->clPlatformName = (gchar*)" ";
    cc->fastRelaxedMath = TRUE;
    cc->forceRecompile = TRUE;

    g->config->silent = TRUE;

    g->feed_layers = dR_list_createEmptyList();
    g->output_layers = dR_list_createEmptyList();
    g->allNodes = dR_list_createEmptyList();
    g->drViewHandlers = dR_list_createEmptyList();
    g->debugLayer = -1;     // the reference leaves this uninitialised; -1 = no debug download
    return g;
}

void dR_config(dR_Graph* net, gchar* platformname, gboolean silent, gboolean debuginfo,
               gboolean profileGPU, gboolean profileCPU, gchar* temppath) {
    net->clConfig->clPlatformName = platformname ? strdup(platformname) : NULL;
    net->config->silent = silent;
    net->config->debugInfo = debuginfo;
    net->config->profilingCPU = profileCPU;
    net->config->profilingGPU = profileGPU;
    net->config->modelPath = temppath;
}

// Bring up the HIP device and the graph's stream.  Idempotent.
static gboolean ensure_device(dR_Graph* net) {
    dR_ClConfig* cc = net->clConfig;
    if (cc->clContext) return TRUE;
    drhip_device_info info;
    if (device_failed(net, drhip_init((int)cc->clDeviceNumber, &info), "dR_initCL")) return FALSE;
    if (!cc->hipStream) {
        if (device_failed(net, drhip_stream_create(&cc->hipStream), "dR_initCL(stream)")) return FALSE;
        cc->hipOwnsStream = TRUE;
    }
    cc->clCommandQueue = (cl_command_queue)cc->hipStream;
    cc->clDeviceName = fmt_dup("%s (%s)", info.name, info.arch);
    cc->hipNumCU = info.num_cu;
    cc->hipLdsBytes = info.lds_bytes;
    cc->clNumDevices = 1;
    cc->clContext = (cl_context)cc;     // tag: device is up
    if (verbose(net))
        say("deepRACIN HIP device %d: %s, %d CUs, %d KiB LDS/workgroup, %.1f GiB HBM\n", info.device,
            cc->clDeviceName, info.num_cu, info.lds_bytes / 1024, (double)info.hbm_bytes / (1 << 30));
    return TRUE;
}

// (TRUE on purpose: the reference's Python wrapper reads a bool from this call, see the header)
gboolean dR_initCL(dR_Graph* net) { return ensure_device(net) ? TRUE : FALSE; }

void dR_setClEnvironment(dR_Graph* net, cl_context, cl_platform_id, cl_command_queue clcommandqueue,
                         cl_device_id) {
    // The only thing a HIP caller can share is its stream.
    net->clConfig->hipStream = (void*)clcommandqueue;
    net->clConfig->hipOwnsStream = FALSE;
}

void dR_getClEnvironmentFrom(dR_Graph* net, dR_Graph* from) {
    if (!from || !from->clConfig->clContext) return;
    net->clConfig->hipStream = from->clConfig->hipStream;
    net->clConfig->hipOwnsStream = FALSE;
    net->clConfig->clDeviceNumber = from->clConfig->clDeviceNumber;
}

gboolean dR_setAsOutput(dR_Graph* net, dR_Node* node) {
    if (!node->output) {
        node->output = TRUE;
        dR_list_append(net->output_layers, node);
    }
    return TRUE;
}

gboolean dR_prepare(dR_Graph* net) {
    const bool talk = verbose(net);
    // One dR_prepare per graph: the schedule flags of the nodes, the planned buffers and the uploaded
    // weights of the first call are not rolled back, so a second walk would find every node already
    // queued and schedule nothing.  Refused loudly instead of returning a graph that computes nothing.
    if (net->prepared) {
        say("dR_prepare: this graph has been prepared already; build a new graph (dR_NewGraph) to prepare again.\n");
        return FALSE;
    }
    if (net->scheduledLayers) {     // scheduled, but never usable: a dR_prepare that failed, or dR_propagateShapesAndSchedule called by hand
        say("dR_prepare: this graph has been scheduled before (by a dR_prepare that failed, or by a call of "
            "dR_propagateShapesAndSchedule) and cannot be scheduled a second time; build a new graph (dR_NewGraph).\n");
        return FALSE;
    }
    if (!ensure_device(net)) { say("dR_initCL Failed \n"); return FALSE; }
    net->drGraphOff = FALSE;

    if (talk) say("Propagate shapes and schedule...\n");
    if (!dR_propagateShapesAndSchedule(net)) { say("dR_propagateShapesAndSchedule Failed \n"); return FALSE; }
    if (talk) say("Done.\n");

    if (talk) say("Select kernels...\n");
    if (!dR_generateAndCompileKernels(net)) { say("\ndR_generateAndCompileKernels Failed \n"); return FALSE; }
    if (talk) say("Done.\n");

    if (talk) say("Estimate and allocate buffers...\n");
    if (!dR_estimateAndAllocateBuffers(net)) { say("dR_estimateAndAllocateBuffers Failed \n"); return FALSE; }
    if (talk) say("Done. \n");

    if (talk) say("Fill buffers...\n");
    if (!dR_fillBuffers(net)) { say("dR_fillBuffers Failed \n"); return FALSE; }
    if (device_failed(net, drhip_stream_sync(stream_of(net)), "dR_prepare(sync)")) return FALSE;
    if (talk) say("Done.\n\n");

    // pinned staging for the per-image copies, sized for the largest feed node (DR_STAGING=0: plain blocking copies)
    const char* stagingEnv = getenv("DR_STAGING");
    if (!net->drStaging && !(stagingEnv && strcmp(stagingEnv, "0") == 0)) {
        size_t largest = 0;
        for (dR_Node* f : nodes_of(net->feed_layers))
            largest = std::max(largest, (size_t)f->oshape.s0 * f->oshape.s1 * f->oshape.s2 * sizeof(float));
        if (largest > 0 && largest <= ((size_t)64 << 20) && drhip_staging_create(&net->drStaging, largest) != DRHIP_OK)
            net->drStaging = NULL;      // not fatal: the blocking copies still work
    }

    net->prepared = TRUE;
    if (net->config->profilingGPU) {
        say("\nGPU Profiling: Whole graph GPU memory consumption: %4.6f MB \n\n",
            (double)net->clConfig->memConsumptionGPU / 1048576.0);
        net->clConfig->totalKernelGPUTime = 0;
    }
    return TRUE;
}

gint dR_getOutputBuffers(dR_Graph* net, cl_mem** outptr) {
    if (!net->prepared) {
        say("dR_Graph must be prepared before having output buffers. Call dR_prepare first! \n");
        return 0;
    }
    int n = 0;
    for (dR_ListElement* e = net->output_layers->first; e && n < 10; e = e->next)
        outptr[n++] = ((dR_Node*)e->element)->outputBuf->bufptr;
    return n;
}

void dR_feedData(dR_Graph* net, dR_Node* feednode, gfloat* data, gint offset, gint numfloats) {
    if (!feednode || !feednode->outputBuf || offset < 0 || numfloats < 0) {
        say("dR_feedData: feed node has no buffer yet (call dR_prepare first) or bad range\n");
        return;
    }
    // Per-image path: through the graph's pinned staging area, without waiting for the bus.  The caller's
    // array has been read when this returns (as with the reference's blocking write, src/deepRACIN.c:76);
    // the transfer itself is ordered on the graph's stream before the next dR_apply.
    const size_t bytes = (size_t)numfloats * sizeof(float);
    if (net->drStaging && data && bytes <= drhip_staging_upload_capacity(net->drStaging)) {
        device_failed(net, drhip_upload_staged(net->drStaging, (void*)feednode->outputBuf->buf, (size_t)offset * sizeof(float), data, bytes,
                                               stream_of(net)), "dR_feedData");
        return;
    }
    dR_uploadArray(net, (gchar*)"", data, (size_t)offset * sizeof(float), bytes, feednode->outputBuf->buf);
}

// One forward pass: walks the schedule and lets every node enqueue its kernels.  Asynchronous
// unless profiling is enabled (reference src/deepRACIN.c:204-270: clFlush only).  With DR_HIPGRAPH=1
// in the environment the first plain pass records the node walk into a hipGraph and later passes
// replay it with a single launch (not with profilingGPU, a debug layer, or a node whose compute()
// cannot be captured because it blocks or allocates).  Off by default: enqueueing a node costs the
// host 2.5-3 us, less than the shortest kernels take, and kernels enqueued one by one follow each
// other more closely on the device than the kernel nodes of a replayed graph (SqueezeNet 81.8 against
// 87.5 us per pass, VGG16 287.2 against 291.4 us, first result of a single pass 8 us sooner).
//
// profilingGPU: the reference waits for every kernel and reads its cl_event (src/dR_clwrap.c:970-1049).
// Here every kernel launch of the pass carries its own start/stop events while the pass is enqueued
// without waiting; after the last node the pass is awaited once, a node's device time
// (node->drLastKernelMs) is the sum over its kernels, and their sum goes to
// clConfig->totalKernelGPUTime, printed like the reference does.
// Fusions decided by the buffer planner leave some nodes without a stored tensor of their own.
static bool tensor_fused_away(const dR_Node* n) {
    if (n->type == tConv2d) {
        const dR_Conv2d_Data* c = (const dR_Conv2d_Data*)n->layer;
        return c->drFusedPool || c->drFusedAvgPool;
    }
    if (n->type == tPooling && ((const dR_Pooling_Data*)n->layer)->drFused && n->next_layers && n->next_layers->length == 1) {
        const dR_Node* c = (const dR_Node*)n->next_layers->first->element;
        return c->type == tConv2d && ((const dR_Conv2d_Data*)c->layer)->drPooledInput == n;
    }
    if (n->type == tFullyConnected) return ((const dR_FC_Data*)n->layer)->drDeferReduce && !n->output;
    return false;
}

gboolean dR_apply(dR_Graph* net) {
    if (!net->prepared) { say("dR_apply: graph is not prepared. Call dR_prepare first! \n"); return FALSE; }
    dR_ClConfig* cc = net->clConfig;
    const bool profGPU = net->config->profilingGPU, profCPU = net->config->profilingCPU;
    if (net->config->debugInfo) say("Applying graph...\n");

    std::chrono::steady_clock::time_point t0;
    if (profCPU) { t0 = std::chrono::steady_clock::now(); net->config->totalNodeCPUTime = 0.0; }

    // On request plain passes are replayed from a hipGraph captured on the first one (for hosts too slow or
    // too busy to enqueue a node in the time the device takes to run it).
    if (!profGPU && net->debugLayer < 0 && !net->drGraphOff) {
        if (!net->drGraphExec) {
            const char* env = getenv("DR_HIPGRAPH");
            if (!env || strcmp(env, "1") != 0 || drhip_graph_capture_begin(cc->hipStream) != DRHIP_OK) {
                net->drGraphOff = TRUE;
            } else {
                const bool recorded = record_forward_pass(net);
                void* exec = NULL;
                const int rc = drhip_graph_capture_end(cc->hipStream, &exec);
                if (!recorded || rc != DRHIP_OK) {
                    if (exec) drhip_graph_destroy(exec);
                    net->drGraphOff = TRUE;         // a node that cannot be captured: enqueue node by node from now on
                    if (debug(net)) say("dR_apply: forward pass not capturable, running node by node\n");
                } else {
                    net->drGraphExec = exec;
                }
            }
        }
        if (net->drGraphExec) {
            if (device_failed(net, drhip_graph_launch(net->drGraphExec, cc->hipStream), "dR_apply(graph)")) return FALSE;
            if (profCPU) {
                if (device_failed(net, drhip_stream_sync(cc->hipStream), "dR_apply(sync)")) return FALSE;
                double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
                net->drLastApplyMs = ms;
                say("CPU Profiling: Whole graph took: %2.3fms, Sum of all nodes: %2.3fms \n", ms, net->config->totalNodeCPUTime);
            }
            if (net->config->debugInfo) say("Done.\n\n");
            return TRUE;
        }
    }

    // profilingGPU: every kernel launch carries its own start/stop events (drhip_timing_*), and a
    // node's time is the sum of its kernels -- the per-kernel profiling the reference took from
    // OpenCL events (src/dR_clwrap.c:718-741).
    const int nNodes = net->scheduledLayers->length;
    std::vector<int> firstLaunch;
    if (profGPU) { firstLaunch.reserve((size_t)nNodes + 1); drhip_timing_begin(); }

    for (dR_ListElement* e = net->scheduledLayers->first; e; e = e->next) {
        dR_Node* node = (dR_Node*)e->element;
        if (profGPU) firstLaunch.push_back(drhip_timing_count());
        if (!node->compute(net, node)) {
            say("Execution of layer %d failed \n", node->layerID);
            if (profGPU) drhip_timing_end(NULL, 0, NULL);
            return FALSE;
        }
        if (node->layerID == net->debugLayer && net->hostDebugBuffer) {
            if (tensor_fused_away(node))
                say("dR_apply: layer %d is computed inside a neighbouring kernel and its tensor is never stored; set "
                    "debugLayer before dR_prepare and the buffer planner keeps it.\n", node->layerID);
            else
                dR_downloadArray(net, (gchar*)"", node->outputBuf->bufptr, 0,
                                 (size_t)node->oshape.s0 * node->oshape.s1 * sizeof(float), net->hostDebugBuffer);
        }
    }
    if (profGPU) {
        firstLaunch.push_back(drhip_timing_count());
        std::vector<float> ms((size_t)firstLaunch.back() + 1);
        int launches = 0;
        if (device_failed(net, drhip_timing_end(ms.data(), (int)ms.size(), &launches), "dR_apply(profile)")) return FALSE;
        int pos = 0;
        cc->totalKernelGPUTime = 0;
        for (dR_ListElement* e = net->scheduledLayers->first; e; e = e->next, ++pos) {
            float sum = 0.f;
            for (int k = firstLaunch[pos]; k < firstLaunch[pos + 1]; ++k) sum += ms[k];
            ((dR_Node*)e->element)->drLastKernelMs = sum;
            cc->totalKernelGPUTime += sum;
        }
        say("GPU Profiling: Sum of all kernel run times: %2.3fms \n", cc->totalKernelGPUTime);   // unconditional, like the reference
        cc->sumTotalKernelGPUTime += cc->totalKernelGPUTime;
        if (cc->totalKernelGPUTime > cc->maxTotalKernelGPUTime) cc->maxTotalKernelGPUTime = cc->totalKernelGPUTime;
        cc->queueKernelGPUTime = cc->totalKernelGPUTime;   // last pass, kept after the running sum is reset
        cc->totalKernelGPUTime = 0;
    }
    if (profCPU) {
        if (device_failed(net, drhip_stream_sync(cc->hipStream), "dR_apply(sync)")) return FALSE;
        double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        net->drLastApplyMs = ms;
        say("CPU Profiling: Whole graph took: %2.3fms, Sum of all nodes: %2.3fms \n", ms, net->config->totalNodeCPUTime);
    }
    if (net->config->debugInfo) say("Done.\n\n");
    return TRUE;
}

void dR_cleanup(dR_Graph* net, gboolean cleanupcl) {
    const bool talk = verbose(net);
    if (talk) say("Cleaning up deepRACIN...\n");
    if (net->clConfig->clContext) {
        drhip_stream_sync(net->clConfig->hipStream);
        unsigned late = 0;      // joined Winograd splits whose partner never delivered (their outputs were set to NaN)
        if (net->prepared && drhip_conv3x3_winograd_join_timeouts(&late) == DRHIP_OK && late > 0)
            say("deepRACIN: %u partial tiles of split convolutions never arrived in this process (device shared with other work?); "
                "the affected outputs were NaN. DR_WINO_JOIN=0 selects the two-kernel form.\n", late);
    }
    if (net->drGraphExec) { drhip_graph_destroy(net->drGraphExec); net->drGraphExec = NULL; }
    if (net->drStaging) { drhip_staging_destroy(net->drStaging); net->drStaging = NULL; }
    for (int k = 0; k < 4; ++k) { drhip_event_destroy(net->drBranchEvents[k]); net->drBranchEvents[k] = NULL; }
    for (int k = 0; k < 3; ++k) { drhip_stream_destroy(net->drSideStreams[k]); net->drSideStreams[k] = NULL; }
    if (net->prepared) dR_cleanupBuffers(net);
    if (cleanupcl) dR_cleanupCL(net);
    dR_cleanupNet(net);
    if (talk) say("Done.\n");
}

gboolean dR_cleanupCL(dR_Graph* net) {
    dR_ClConfig* cc = net->clConfig;
    if (!cc->clContext || cc->cleanupDone) return TRUE;
    if (cc->hipOwnsStream && cc->hipStream) drhip_stream_destroy(cc->hipStream);
    cc->hipStream = NULL;
    free(cc->clDeviceName);
    cc->clDeviceName = NULL;
    cc->clContext = NULL;
    cc->cleanupDone = TRUE;
    return TRUE;
}

gboolean dR_saveGraph(dR_Graph* net, gchar* path) { return dR_serializeGraph(net, path); }

dR_Node* dR_loadGraph(dR_Graph* net, gchar* path, dR_Node*** nodelist, gint* numnodes,
                      dR_Node*** feednodes, gint* numfeednodes) {
    return dR_parseGraph(net, path, nodelist, numnodes, feednodes, numfeednodes);
}

void dR_printNetObject(dR_Graph* net, char* path) { dR_printNet(net, path); }

dR_Shape3* dR_getOutputShape(dR_Node* node) { return &node->oshape; }

dR_Shape3* dR_getFeedNodeInputShape(dR_Node* node) {
    if (node->type != tDataFeedNode) {
        say("Error: dR_getFeedNodeInputShape only works on feed nodes!\n");
        return NULL;
    }
    return &((dR_DataFeedNode_Data*)node->layer)->shape;
}

// ---- caller-supplied buffers -------------------------------------------------------------------

gboolean dR_setDataFeedNodeBuffer(dR_Graph* net, dR_Node* node, cl_mem* buf) {
    if (node->type != tDataFeedNode) {
        if (verbose(net)) say("dR_setDataFeedNodeBuffer Error: Data Feed Buffer can only be set to a DataFeedNode!\n");
        return FALSE;
    }
    dR_DataFeedNode_Data* feed = (dR_DataFeedNode_Data*)node->layer;
    node->outputBuf = dR_newMemoryHandler(TRUE);
    node->outputBuf->bufptr = buf;
    node->outputBuf->buf = *buf;
    node->outputBuf->size = feed->shape.s0 * feed->shape.s1 * feed->shape.s2;
    dR_list_append(node->outputBuf->outputFor, node);
    return TRUE;
}

gboolean dR_setPreexistingOutputBuffer(dR_Graph* net, dR_Node* node, cl_mem* buf) {
    node->outputBuf = dR_newMemoryHandler(TRUE);
    node->outputBuf->bufptr = buf;
    node->outputBuf->buf = *buf;
    if (!node->output) dR_setAsOutput(net, node);
    return TRUE;
}

// Region-of-interest plumbing belongs to the image-processing nodes, which this build does not carry.
gboolean dR_setNodeRoI(dR_Node*, dR_Shape3) { return FALSE; }
gboolean dR_setNodeRoIBufferAndIndex(dR_Node*, cl_mem*, gint) { return FALSE; }

// ---- device memory helpers (names of the reference's OpenCL wrapper) ------------------------------

gboolean dR_createFloatBuffer(dR_Graph* net, cl_mem* mem, gint size, int /*buffertype*/) {
    if (size <= 0) { say("dR_createFloatBuffer: refusing to allocate %d floats\n", size); return FALSE; }
    void* p = NULL;
    if (device_failed(net, drhip_malloc(&p, (size_t)size * sizeof(float)), "dR_createFloatBuffer")) return FALSE;
    *mem = (cl_mem)p;
    net->clConfig->memConsumptionGPU += (glong)size * (glong)sizeof(float);
    return TRUE;
}

gboolean dR_clMemoryBufferCleanup(dR_Graph* net, cl_mem mem) {
    if (!mem) return TRUE;
    return !device_failed(net, drhip_free((void*)mem), "dR_clMemoryBufferCleanup");
}

gboolean dR_uploadArray(dR_Graph* net, gchar*, void* srcHostMem, size_t offset, size_t numBytes,
                        cl_mem destDeviceMem) {
    if (!destDeviceMem || !srcHostMem) { say("dR_uploadArray: NULL buffer\n"); return FALSE; }
    return !device_failed(net, drhip_upload((void*)destDeviceMem, offset, srcHostMem, numBytes, stream_of(net)),
                          "dR_uploadArray");
}

void dR_downloadArray(dR_Graph* net, gchar*, cl_mem* srcDeviceMem, size_t byteOffset, size_t numBytes,
                      void* destHostMem) {
    if (!srcDeviceMem || !*srcDeviceMem || !destHostMem) { say("dR_downloadArray: NULL buffer\n"); return; }
    if (net->drStaging && numBytes <= drhip_staging_download_capacity(net->drStaging)) {
        device_failed(net, drhip_download_staged(net->drStaging, destHostMem, (const void*)*srcDeviceMem, byteOffset, numBytes, stream_of(net)),
                      "dR_downloadArray");
        return;
    }
    device_failed(net, drhip_download(destHostMem, (const void*)*srcDeviceMem, byteOffset, numBytes, stream_of(net)),
                  "dR_downloadArray");
}

}  // extern "C"
