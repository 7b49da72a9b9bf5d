/*
 * deepRACIN.h -- the deepRacin C graph API, served by hand-written HIP kernels on MI355X (gfx950).
 *
 * Drop-in boundary: every function below keeps the name, argument list and meaning it has in the
 * reference (citations are to the reference tree), so a host program written against deepRacin
 * links against this libdeepracin.so unchanged.  Typical life cycle (reference README.md:64-90):
 *
 *   dR_NewGraph -> [dR_config] -> dR_initCL -> dR_loadGraph | node constructors -> dR_setAsOutput
 *     -> dR_prepare -> dR_getOutputBuffers -> { dR_feedData -> dR_apply -> dR_downloadArray }*
 *     -> dR_cleanup
 *
 * Threading: none. One graph owns one HIP stream; the library is not re-entrant (lists carry one
 * embedded cursor, like the reference).  dR_apply only enqueues; dR_downloadArray, dR_uploadArray
 * and dR_feedData block.  Errors: gboolean FALSE / NULL / 0 plus a message on stdout.
 */
#ifndef DR_H
#define DR_H

#include "dR_types.h"
#include "dR_nodes.h"
#include "dr_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------------------------------------
 * Graph life cycle
 * ------------------------------------------------------------------------------------------- */

/* New empty graph with default configuration: silent, no profiling, device 0.
 * (reference include/deepRACIN.h:18, src/deepRACIN.c:6-47) */
dR_Graph*  dR_NewGraph(void);

/* Set run-time options; temppath becomes config->modelPath.  platformname is accepted and
 * ignored (there is exactly one platform: HIP).  (deepRACIN.h:262, deepRACIN.c:321-335) */
void       dR_config(dR_Graph* net, gchar* platformname, gboolean silent, gboolean debuginfo,
                     gboolean profileGPU, gboolean profileCPU, gchar* temppath);

/* Bring up the device: selects HIP device clConfig->clDeviceNumber, creates the graph's stream.
 * Keeps its OpenCL-era name.  dR_prepare calls it implicitly if the caller did not.
 * Returns TRUE when the device is up.  The reference declares this function void (deepRACIN.h:155,
 * deepRACIN.c:144-146), yet its own Python wrapper binds it with a bool result and refuses to go on when
 * that is false (python/deepracin/__init__.py.in:55-58, 422-426): there the TRUE of dR_clInit happens to be
 * left in the return register.  Here the result is returned on purpose; a C caller written against the
 * void declaration ignores it. */
gboolean   dR_initCL(dR_Graph* net);

/* Mark a node whose buffer must survive dR_apply and be retrievable with dR_getOutputBuffers.
 * (deepRACIN.h:142, deepRACIN.c:133-141) */
gboolean   dR_setAsOutput(dR_Graph* net, dR_Node* node);

/* Shape propagation + gfx950 scheduling, buffer planning and allocation, weight upload.
 * Needs >= 1 feed node.  (deepRACIN.h:182, deepRACIN.c:148-202) */
gboolean   dR_prepare(dR_Graph* net);

/* Write up to 10 pointers-to-handle of the output nodes' buffers, in dR_setAsOutput order, into
 * outptr; returns how many; 0 with a message if the graph is not prepared.  The handles stay
 * owned by the graph and valid until dR_cleanup.  (deepRACIN.h:32, deepRACIN.c:51-72) */
gint       dR_getOutputBuffers(dR_Graph* net, cl_mem** outptr);

/* Host->device copy of numfloats floats into the feed node's buffer, starting at float index offset.
 * The caller's array has been read when the call returns (it may be reused at once, as after the
 * reference's blocking write); the transfer itself is asynchronous, from a pinned staging area the graph
 * owns, ordered on the graph's stream in front of the next dR_apply.  Arrays larger than the staging area
 * (sized at dR_prepare for the largest feed node) and DR_STAGING=0 take a blocking copy.
 * (deepRACIN.h:47, deepRACIN.c:74-77) */
void       dR_feedData(dR_Graph* net, dR_Node* feednode, gfloat* data, gint offset, gint numfloats);

/* Enqueue one forward pass on the graph's stream; returns without waiting unless profiling is on.
 * (deepRACIN.h:169, deepRACIN.c:204-270) */
gboolean   dR_apply(dR_Graph* net);

/* Release device buffers, nodes and the graph; cleanupcl also destroys the stream.
 * (deepRACIN.h:194, deepRACIN.c:272-282) */
void       dR_cleanup(dR_Graph* net, gboolean cleanupcl);

/* ---------------------------------------------------------------------------------------------
 * Stored graph format (graph.dr + N.var), byte compatible with the reference
 * ------------------------------------------------------------------------------------------- */

/* Writes <path>/dr_graph_export/graph.dr and one raw little-endian fp32 file per variable.
 * (deepRACIN.h:213, src/dR_parser.c:58-180) */
gboolean   dR_saveGraph(dR_Graph* net, gchar* path);

/* Reads <path>/graph.dr into an EMPTY graph.  *nodelist / *feednodes are malloc'ed arrays handed
 * to the caller (free() them); returns the last node, NULL on any error.
 * (deepRACIN.h:216, src/dR_parser.c:182-523) */
dR_Node*   dR_loadGraph(dR_Graph* net, gchar* path, dR_Node*** nodelist, gint* numnodes,
                        dR_Node*** feednodes, gint* numfeednodes);

/* Human-readable dump of all nodes to stdout (path == NULL) or to a file.  (deepRACIN.h:227) */
void       dR_printNetObject(dR_Graph* net, char* path);

/* ---------------------------------------------------------------------------------------------
 * Shapes
 * ------------------------------------------------------------------------------------------- */
dR_Shape3* dR_getOutputShape(dR_Node* node);            /* pointer into the node  (deepRACIN.h:279) */
dR_Shape3* dR_getFeedNodeInputShape(dR_Node* node);     /* NULL unless a feed node (deepRACIN.h:57)  */

/* ---------------------------------------------------------------------------------------------
 * Buffer sharing entry points.  In the reference these share OpenCL objects with the caller; here
 * the handles are HIP device addresses (see dr_compat.h).
 * ------------------------------------------------------------------------------------------- */
/* Use the caller's device buffer (*clbuf = device address) as the feed node's storage. (deepRACIN.h:72) */
gboolean   dR_setDataFeedNodeBuffer(dR_Graph* net, dR_Node* feednode, cl_mem* clbuf);
/* Make the node write into the caller's device buffer and mark it as output.          (deepRACIN.h:126) */
gboolean   dR_setPreexistingOutputBuffer(dR_Graph* net, dR_Node* node, cl_mem* buf);
/* Region-of-interest hooks of nodes outside the CNN layer path: accepted, return FALSE. (deepRACIN.h:90,108) */
gboolean   dR_setNodeRoI(dR_Node* node, dR_Shape3 origin);
gboolean   dR_setNodeRoIBufferAndIndex(dR_Node* node, cl_mem* buf, gint index);
/* Adopt a caller-owned stream: clcommandqueue is taken as a hipStream_t, the other handles are
 * ignored.  (deepRACIN.h:242, deepRACIN.c:304-315) */
void       dR_setClEnvironment(dR_Graph* net, cl_context clcontext, cl_platform_id clplatformid,
                               cl_command_queue clcommandqueue, cl_device_id cldeviceid);
/* Share the stream of an already initialised graph (called by the reference's Python wrapper,
 * python/deepracin/__init__.py.in:428, although the reference never defines it). */
void       dR_getClEnvironmentFrom(dR_Graph* net, dR_Graph* from);

/* ---------------------------------------------------------------------------------------------
 * Device memory helpers kept from the OpenCL wrapper (reference include/dR_clwrap.h:20,34,45)
 * ------------------------------------------------------------------------------------------- */
/* Blocking H2D copy of numBytes to byte offset `offset` of destDeviceMem. */
gboolean   dR_uploadArray(dR_Graph* net, gchar* name, void* srcHostMem, size_t offset,
                          size_t numBytes, cl_mem destDeviceMem);
/* Blocking D2H copy; this is the synchronisation point after dR_apply. */
void       dR_downloadArray(dR_Graph* net, gchar* name, cl_mem* srcDeviceMem, size_t byteOffset,
                            size_t numBytes, void* destHostMem);
/* Allocate `size` floats of device memory; buffertype (CL_MEM_*) is accepted and ignored. */
gboolean   dR_createFloatBuffer(dR_Graph* net, cl_mem* mem, gint size, int buffertype);
gboolean   dR_clMemoryBufferCleanup(dR_Graph* net, cl_mem mem);
gboolean   dR_cleanupCL(dR_Graph* net);

/* ---------------------------------------------------------------------------------------------
 * Graph core, exported for custom node plug-ins (reference include/dR_core.h)
 * ------------------------------------------------------------------------------------------- */
dR_Node*   dR_Datafeednode(dR_Graph* net, dR_Shape3* shape);         /* dR_core.h:39 */
dR_Graph*  dR_appendLayer(dR_Graph* net, dR_Node* l);                /* assigns layerID, registers the node */
gboolean   dR_propagateShapesAndSchedule(dR_Graph* net);             /* src/dR_core.c:121-211 */
gboolean   dR_generateAndCompileKernels(dR_Graph* net);              /* :371-418; here: createKernel hooks only */
gboolean   dR_estimateAndAllocateBuffers(dR_Graph* net);             /* :213-325 */
gboolean   dR_fillBuffers(dR_Graph* net);                            /* :328-341 */
void       dR_cleanupBuffers(dR_Graph* net);
void       dR_cleanupNet(dR_Graph* net);
dR_MemoryHandler* dR_newMemoryHandler(gboolean custom);
void       dR_cleanupMemoryHandler(dR_Graph* net, dR_MemoryHandler* handler);
/* Buffer plan without touching the device: fills every node's outputBuf (sizes, aliasing, views)
 * but allocates nothing.  dR_estimateAndAllocateBuffers = this + allocation.  Lets the planner be
 * checked on a machine without a GPU. */
gboolean   dR_planBuffers(dR_Graph* net);

dR_List*   dR_list_createEmptyList(void);
void       dR_list_append(dR_List* list, void* elem);
gboolean   dR_list_removeFirstOcc(dR_List* list, void* elem);
void*      dR_list_pop(dR_List* list);
void*      dR_list_next(dR_List* list);
void       dR_list_resetIt(dR_List* list);
void       dR_list_cleanup(dR_List* list);

/* result = mat1 (r1 x c1) * mat2 (r2 x c2) and mat1 * mat2^T, naive fp32 loops (src/dR_core.c:677-723). */
gboolean   dR_matmul(gfloat* mat1, gint mat1rows, gint mat1cols, gfloat* mat2, gint mat2rows,
                     gint mat2cols, gfloat* result);
gboolean   dR_matmulT(gfloat* mat1, gint mat1rows, gint mat1cols, gfloat* mat2, gint mat2rows,
                      gint mat2cols, gfloat* result);

gboolean   dR_serializeGraph(dR_Graph* net, gchar* path);            /* src/dR_parser.c:58 */
dR_Node*   dR_parseGraph(dR_Graph* net, gchar* path, dR_Node*** nodelist, gint* numnodes,
                         dR_Node*** feednodes, gint* numfeednodes);  /* src/dR_parser.c:182 */
void       dR_printNet(dR_Graph* net, char* path);
void       dR_printSchedule(dR_Graph* net);

#ifdef __cplusplus
}
#endif
#endif /* DR_H */
