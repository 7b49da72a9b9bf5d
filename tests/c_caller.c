/*
 * A host program in plain C against the public headers, in the shape of the reference's own example
 * (examples/squeezenet-v1.1/squeezenet_deployed.c:92-227): it reaches into net->config and net->clConfig,
 * loads a stored model, marks the last node as output, prepares, and then feeds / applies / downloads
 * once per image and prints the class with the largest probability.
 *
 *     c_caller <model directory> <image.f32> [<image.f32> ...]
 *
 * An image file holds 224*224*3 raw floats in [c][h][w] order (the test writes them; the reference's example
 * reads PNGs with libpng and swaps the axes itself).  Output: one line "class <n>" per image.
 *
 * The _Static_assert block pins this library's struct layouts to the reference's include/dR_types.h: a program
 * compiled against the reference's headers finds every field it may touch at the same offset
 * (tests/golden/ref_struct_offsets.h holds the reference's numbers).
 */
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>

#include "deepRACIN.h"
#include "golden/ref_struct_offsets.h"

#define SAME(S, F) _Static_assert(offsetof(S, F) == REF_OFFSETOF_##S##_##F, #S "." #F " is not where the reference has it")
#define SAME_SIZE(S) _Static_assert(sizeof(S) == REF_SIZEOF_##S, "sizeof(" #S ") differs from the reference's")
#define AT_LEAST(S) _Static_assert(sizeof(S) >= REF_SIZEOF_##S, #S " is smaller than the reference's")

SAME_SIZE(dR_Shape2); SAME(dR_Shape2, s0); SAME(dR_Shape2, s1);
SAME_SIZE(dR_Shape3); SAME(dR_Shape3, s0); SAME(dR_Shape3, s1); SAME(dR_Shape3, s2);
SAME_SIZE(dR_Shape4); SAME(dR_Shape4, s0); SAME(dR_Shape4, s1); SAME(dR_Shape4, s2); SAME(dR_Shape4, s3);
SAME_SIZE(dR_Config);
SAME(dR_Config, silent); SAME(dR_Config, profilingGPU); SAME(dR_Config, profilingCPU); SAME(dR_Config, debugInfo);
SAME(dR_Config, totalNodeCPUTime); SAME(dR_Config, convLocalWorkSizeWindow); SAME(dR_Config, modelPath);
AT_LEAST(dR_ClConfig);      /* (fields of this build are appended behind the reference's) */
SAME(dR_ClConfig, clContext); SAME(dR_ClConfig, clPlatformId); SAME(dR_ClConfig, clCommandQueue); SAME(dR_ClConfig, clProgram);
SAME(dR_ClConfig, clDeviceType); SAME(dR_ClConfig, clDeviceNumber); SAME(dR_ClConfig, clPlatformName); SAME(dR_ClConfig, clKernelPath);
SAME(dR_ClConfig, clDeviceId); SAME(dR_ClConfig, clNumDevices); SAME(dR_ClConfig, clDeviceIds); SAME(dR_ClConfig, clDeviceName);
SAME(dR_ClConfig, clError); SAME(dR_ClConfig, clEventObject); SAME(dR_ClConfig, clEvent); SAME(dR_ClConfig, forceRecompile);
SAME(dR_ClConfig, totalKernelGPUTime); SAME(dR_ClConfig, queueKernelGPUTime); SAME(dR_ClConfig, maxTotalKernelGPUTime);
SAME(dR_ClConfig, sumTotalKernelGPUTime); SAME(dR_ClConfig, clInfo); SAME(dR_ClConfig, fastRelaxedMath); SAME(dR_ClConfig, build_status);
SAME(dR_ClConfig, cleanupDone); SAME(dR_ClConfig, configH); SAME(dR_ClConfig, memConsumptionGPU);
AT_LEAST(dR_Graph);
SAME(dR_Graph, prepared); SAME(dR_Graph, swapBuffer1); SAME(dR_Graph, swapBuffer2); SAME(dR_Graph, config); SAME(dR_Graph, clConfig);
SAME(dR_Graph, feed_layers); SAME(dR_Graph, output_layers); SAME(dR_Graph, streamBufferHandlers); SAME(dR_Graph, number_of_layers);
SAME(dR_Graph, maxBufferSize); SAME(dR_Graph, hostDebugBuffer); SAME(dR_Graph, scheduledLayers); SAME(dR_Graph, allNodes);
SAME(dR_Graph, debugLayer);
AT_LEAST(dR_Node);
SAME(dR_Node, oshape); SAME(dR_Node, layerID); SAME(dR_Node, previous_layers); SAME(dR_Node, next_layers); SAME(dR_Node, clKernel);
SAME(dR_Node, outputBuf); SAME(dR_Node, layer); SAME(dR_Node, type); SAME(dR_Node, propagated); SAME(dR_Node, output); SAME(dR_Node, queued);
SAME(dR_Node, compute); SAME(dR_Node, schedule); SAME(dR_Node, propagateShape); SAME(dR_Node, getRequiredOutputBufferSize);
SAME(dR_Node, createKernel); SAME(dR_Node, allocateBuffers); SAME(dR_Node, fillBuffers); SAME(dR_Node, cleanupBuffers);
SAME(dR_Node, cleanupLayer); SAME(dR_Node, printLayer); SAME(dR_Node, serializeNode); SAME(dR_Node, parseAppendNode);
SAME(dR_Node, generateKernel); SAME(dR_Node, createKernelName); SAME(dR_Node, setVariables);
AT_LEAST(dR_MemoryHandler);
SAME(dR_MemoryHandler, outputFor); SAME(dR_MemoryHandler, size); SAME(dR_MemoryHandler, numberOfDependencies); SAME(dR_MemoryHandler, bufptr);
SAME(dR_MemoryHandler, buf); SAME(dR_MemoryHandler, outputBuf); SAME(dR_MemoryHandler, regionOfInterest);
SAME(dR_MemoryHandler, useIndexBufferForRoI); SAME(dR_MemoryHandler, indexBuffer); SAME(dR_MemoryHandler, index); SAME(dR_MemoryHandler, roiOrigin);
SAME_SIZE(dR_ListElement); SAME(dR_ListElement, next); SAME(dR_ListElement, previous); SAME(dR_ListElement, element);
SAME_SIZE(dR_List); SAME(dR_List, first); SAME(dR_List, last); SAME(dR_List, length); SAME(dR_List, iterator);

enum { width = 224, height = 224, classes = 1000 };

static int read_image(const char* path, float* dst, size_t n) {
    FILE* fp = fopen(path, "rb");
    if (!fp) { fprintf(stderr, "c_caller: cannot open %s\n", path); return 0; }
    const size_t got = fread(dst, sizeof(float), n, fp);
    fclose(fp);
    if (got != n) { fprintf(stderr, "c_caller: %s holds %zu floats, expected %zu\n", path, got, n); return 0; }
    return 1;
}

int main(int argc, char** argv) {
    if (argc < 3) { fprintf(stderr, "usage: %s <model directory> <image.f32> ...\n", argv[0]); return 2; }
    const int buffersize = width * height * 3 * (int)sizeof(float);
    float* feed_buffer = (float*)malloc((size_t)buffersize);

    dR_Graph* net;
    dR_Node** feedlist;
    dR_Node** nodeslist;
    gint numnodes;
    gint numfeeds;
    dR_Node* lastnode;

    net = dR_NewGraph();
    /* the switches the reference's example sets by reaching into the structs */
    net->config->debugInfo = FALSE;
    net->config->profilingGPU = TRUE;
    net->config->profilingCPU = TRUE;
    net->config->silent = TRUE;
    net->clConfig->clPlatformName = NULL;
    dR_initCL(net);

    if (!dR_loadGraph(net, argv[1], &nodeslist, &numnodes, &feedlist, &numfeeds) || numfeeds < 1) {
        fprintf(stderr, "c_caller: loading %s failed\n", argv[1]);
        return 1;
    }
    lastnode = nodeslist[numnodes - 1];
    dR_setAsOutput(net, lastnode);
    if (!dR_prepare(net)) { fprintf(stderr, "c_caller: dR_prepare failed\n"); return 1; }

    cl_float* odata = (gfloat*)malloc(classes * sizeof(gfloat));
    cl_mem* outbuffers[1];
    if (dR_getOutputBuffers(net, outbuffers) != 1) { fprintf(stderr, "c_caller: expected one output buffer\n"); return 1; }

    for (int i = 2; i < argc; i++) {
        if (!read_image(argv[i], feed_buffer, (size_t)width * height * 3)) return 1;
        dR_feedData(net, feedlist[0], (cl_float*)feed_buffer, 0, buffersize / (int)sizeof(float));
        if (!dR_apply(net)) { fprintf(stderr, "c_caller: dR_apply failed\n"); return 1; }
        dR_downloadArray(net, (gchar*)"", outbuffers[0], 0, classes * sizeof(cl_float), odata);
        float max = odata[0];
        int argmax = 0;
        for (int j = 0; j < classes; j++)
            if (odata[j] > max) { max = odata[j]; argmax = j; }
        fflush(stdout);     /* (the library prints its profiling lines through its own buffer) */
        printf("class %d\n", argmax);
        fflush(stdout);
    }
    if (net->clConfig->sumTotalKernelGPUTime <= 0.0) { fprintf(stderr, "c_caller: profilingGPU left no kernel time behind\n"); return 1; }

    free(feed_buffer);
    free(odata);
    dR_cleanup(net, TRUE);
    return 0;
}
