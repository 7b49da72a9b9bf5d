/*
 * dR_types.h -- data model of the deepRacin graph API as served by the MI355X (gfx950, HIP) build.
 *
 * Mirrors the public structs of the reference (include/dR_types.h:17-228): field names, order and
 * widths of the reference are kept so that user code which pokes `net->config->silent`,
 * `net->clConfig->clPlatformName`, `node->oshape` ... keeps compiling and keeps its offsets.
 * Fields that only made sense for OpenCL stay as inert placeholders.  Everything this build adds
 * is appended AFTER the reference's last field of each struct and is prefixed `hip`/`dr`.
 *
 * Tensor convention (reference include/deepRACIN.h:61,79): a shape (s0,s1,s2) = (W,H,C) denotes a
 * flat fp32 array in [C][H][W] order, x fastest.
 */
#ifndef DR_TYPES_H
#define DR_TYPES_H

#include "dr_compat.h"
#include <string.h>
#include <stdlib.h>

typedef struct dR_Config            dR_Config;
typedef struct dR_ClConfig          dR_ClConfig;
typedef struct dR_Node              dR_Node;
typedef struct dR_Graph             dR_Graph;
typedef struct dR_ListElement       dR_ListElement;
typedef struct dR_List              dR_List;
typedef struct dR_DataFeedNode_Data dR_DataFeedNode_Data;
typedef struct dR_MemoryHandler     dR_MemoryHandler;
typedef struct dR_Shape2            dR_Shape2;
typedef struct dR_Shape3            dR_Shape3;
typedef struct dR_Shape4            dR_Shape4;

/* ---- shapes -------------------------------------------------------------------------------- */
struct dR_Shape2 { gint s0, s1; };
struct dR_Shape3 { gint s0, s1, s2; };
struct dR_Shape4 { gint s0, s1, s2, s3; };

/* ---- node plug-in interface (reference include/dR_types.h:30-48) ----------------------------
 * A node is a struct of function pointers; dR_prepare drives them in this order:
 *   propagateShape -> schedule -> [generateKernel] -> createKernel -> allocateBuffers -> fillBuffers
 * and dR_apply calls compute() per node in schedule order.  In this build:
 *   schedule()     picks the gfx950 kernel variant and tile parameters (no OpenCL work sizes),
 *   createKernel() is a no-op hook (kernels are compiled ahead of time into the library),
 *   generateKernel() is never needed and may be NULL,
 *   compute()      enqueues hand-written HIP kernels on the graph's stream through drhip_*.
 */
typedef gboolean (*fCompute)         (dR_Graph* net, dR_Node* node);
typedef gboolean (*fSchedule)        (dR_Graph* net, dR_Node* node);
typedef gboolean (*fPropagate)       (dR_Graph* net, dR_Node* node);
typedef gint32   (*fMaxBuffer)       (dR_Node* node);
typedef gboolean (*fCreateKernel)    (dR_Graph* net, dR_Node* node);
typedef gboolean (*fAllocateBuffers) (dR_Graph* net, dR_Node* node);
typedef gboolean (*fFillBuffers)     (dR_Graph* net, dR_Node* node);
typedef gboolean (*fCleanupBuffers)  (dR_Graph* net, dR_Node* node);
typedef gboolean (*fCleanupLayer)    (dR_Graph* net, dR_Node* node);
typedef gchar*   (*fPrintLayer)      (dR_Node* node);
typedef gchar*   (*fSerializeNode)   (dR_Node* node, gchar* params[], gint* numParams,
                                      gfloat* variables[], gint variableSizes[], gint* numVariables);
typedef dR_Node* (*fParseAppendNode) (dR_Graph* net, dR_Node** iNodes, gint numINodes,
                                      gchar** params, gint numParams,
                                      gfloat** variables, gint numVariables);
typedef gboolean (*fGenerateKernel)  (dR_Graph* net, dR_Node* node);
typedef gchar*   (*fCreateKernelName)(dR_Node* node);
typedef void     (*fSetVariables)    (dR_Node* node, gfloat* weights, gfloat* bias);

/* Node kinds; numeric values are those of the reference (include/dR_types.h:73-95). */
enum dR_LayerType {
    tPooling, tBN, tFullyConnected, tConv2d, tPPFilter, tMaskDependentFilter, tLabelCreation,
    tNormalization, tUpscaling, tRGB2Gray, tMulScalar, tAddScalar, tDataFeedNode, tResolveRoI,
    tSoftmax, tSlice, tConcat, tCropOrPad, tElemWise2Op, tElemWise1Op, tFFT
};
typedef enum dR_LayerType dR_LayerType;

/* Activation selector stored in graph.dr (0 linear, 1 ReLU; 2/3 are unimplemented upstream too). */
enum dR_ActivationType { tLinear, tReLU, tSigmoid, tTan };
typedef enum dR_ActivationType dR_ActivationType;

struct dR_DataFeedNode_Data {
    dR_Shape3   shape;          /* (W,H,C) of the fed tensor */
    cl_mem      dataBuffer;
    dR_List*    next_layers;
};

struct dR_Node {
    dR_Shape3           oshape;             /* output (W,H,C), valid after propagateShape */
    gint32              layerID;            /* creation index == id used in graph.dr */
    dR_List*            previous_layers;
    dR_List*            next_layers;
    cl_kernel           clKernel;           /* unused placeholder */
    dR_MemoryHandler*   outputBuf;
    void*               layer;              /* node-type specific data (dR_Conv2d_Data, ...) */
    dR_LayerType        type;
    gboolean            propagated;
    gboolean            output;
    gboolean            queued;

    fCompute            compute;
    fSchedule           schedule;
    fPropagate          propagateShape;
    fMaxBuffer          getRequiredOutputBufferSize;
    fCreateKernel       createKernel;
    fAllocateBuffers    allocateBuffers;
    fFillBuffers        fillBuffers;
    fCleanupBuffers     cleanupBuffers;
    fCleanupLayer       cleanupLayer;
    fPrintLayer         printLayer;
    fSerializeNode      serializeNode;
    fParseAppendNode    parseAppendNode;

    fGenerateKernel     generateKernel;
    fCreateKernelName   createKernelName;
    fSetVariables       setVariables;

    /* ---- additions of this build ---- */
    gint                drSchedulePos;      /* index in net->scheduledLayers, -1 for feed nodes */
    gfloat              drLastKernelMs;     /* device time of the last compute() when profilingGPU */
};

struct dR_ClConfig {
    cl_context          clContext;          /* non-NULL once dR_initCL succeeded (a tag, not a CL object) */
    cl_platform_id      clPlatformId;
    cl_command_queue    clCommandQueue;     /* the graph's hipStream_t, cast */
    cl_program          clProgram;
    cl_uint             clDeviceType;
    cl_uint             clDeviceNumber;     /* HIP device ordinal */
    gchar*              clPlatformName;     /* accepted, ignored */
    gchar*              clKernelPath;       /* accepted, ignored: kernels are built into the library */
    cl_device_id        clDeviceId;
    cl_uint             clNumDevices;
    cl_device_id        clDeviceIds[20];
    gchar*              clDeviceName;       /* e.g. "AMD Instinct MI355X (gfx950)" */
    cl_int              clError;            /* last drhip_* status, 0 = success */
    cl_event            clEventObject;
    cl_event*           clEvent;
    gboolean            forceRecompile;
    gdouble             totalKernelGPUTime; /* ms, summed over the nodes of the running dR_apply */
    gdouble             queueKernelGPUTime;
    gdouble             maxTotalKernelGPUTime;
    gdouble             sumTotalKernelGPUTime;
    gboolean            clInfo;
    gboolean            fastRelaxedMath;
    cl_build_status     build_status;
    gboolean            cleanupDone;
    gchar*              configH;
    glong               memConsumptionGPU;  /* bytes of device memory held by the graph */

    /* ---- additions of this build ---- */
    void*               hipStream;          /* hipStream_t all work of this graph is ordered on */
    gint                hipNumCU;           /* compute units of the device (256 on MI355X) */
    gint                hipLdsBytes;        /* LDS bytes per workgroup limit */
    gboolean            hipOwnsStream;
};

struct dR_Config {
    gboolean    silent;
    gboolean    profilingGPU;               /* per-node hipEvent timing; dR_apply then waits for the pass to finish */
    gboolean    profilingCPU;               /* wall clock around the whole dR_apply incl. a final sync */
    gboolean    debugInfo;
    gdouble     totalNodeCPUTime;
    gint        convLocalWorkSizeWindow;
    gchar*      modelPath;
};

struct dR_Graph {
    gboolean        prepared;
    cl_mem          swapBuffer1;
    cl_mem          swapBuffer2;
    dR_Config*      config;
    dR_ClConfig*    clConfig;
    dR_List*        feed_layers;
    dR_List*        output_layers;
    dR_List*        streamBufferHandlers;
    gint32          number_of_layers;
    gint32          maxBufferSize;
    cl_float*       hostDebugBuffer;
    dR_List*        scheduledLayers;
    dR_List*        allNodes;
    gint            debugLayer;

    /* ---- additions of this build ---- */
    dR_List*        drViewHandlers;         /* handlers that alias a slice of a stream buffer */
    gdouble         drLastApplyMs;          /* wall ms of the last dR_apply when profilingCPU */
    void*           drGraphExec;            /* hipGraphExec_t of the captured forward pass, NULL until captured */
    gboolean        drGraphOff;             /* TRUE: always enqueue node by node (DR_HIPGRAPH=1 not set, or capture failed) */
    void*           drSideStreams[3];       /* streams that carry independent sibling nodes inside the captured graph */
    void*           drBranchEvents[4];      /* fork event [0] and join events [1..3] of a sibling group */
    gint            drBranchGroups;         /* number of sibling groups the captured graph runs concurrently */
    void*           drStaging;              /* pinned staging areas for dR_feedData / dR_downloadArray (drhip_staging_create), made by dR_prepare */
};

struct dR_MemoryHandler {
    dR_List*            outputFor;
    gint                size;                   /* floats */
    gint                numberOfDependencies;
    cl_mem*             bufptr;
    cl_mem              buf;
    gboolean            outputBuf;              /* TRUE: buffer supplied by the caller, never freed here */
    gboolean            regionOfInterest;
    gboolean            useIndexBufferForRoI;
    cl_mem*             indexBuffer;
    gint                index;
    dR_Shape3           roiOrigin;

    /* ---- additions of this build ---- */
    dR_MemoryHandler*   drViewOf;               /* non-NULL: this handler is a window into drViewOf->buf */
    gint                drViewOffset;           /* window start, in floats */
    gint                drFirstDef;             /* schedule position of the first writer */
    gint                drLastUse;              /* schedule position of the last reader */
    gboolean            drPinned;               /* feed / output storage: never recycled */
};

/* ---- intrusive list with one embedded cursor (reference include/dR_types.h:217-228) --------- */
struct dR_ListElement {
    dR_ListElement* next;
    dR_ListElement* previous;
    void*           element;
};

struct dR_List {
    dR_ListElement* first;
    dR_ListElement* last;
    gint            length;
    dR_ListElement* iterator;
};

/* device-type selectors kept for source compatibility */
#define DEVICE_TYPE_DEFAULT     (1 << 0)
#define DEVICE_TYPE_CPU         (1 << 1)
#define DEVICE_TYPE_GPU         (1 << 2)
#define DEVICE_TYPE_ACCELERATOR (1 << 3)
#define DEVICE_TYPE_ALL         0xFFFFFFFF

#endif /* DR_TYPES_H */
