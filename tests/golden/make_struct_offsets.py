"""Writes tests/golden/ref_struct_offsets.h: sizes and field offsets of the structs a host program written
against the reference reaches into (dR_Graph, dR_Config, dR_ClConfig, dR_Node, dR_MemoryHandler, dR_List,
dR_ListElement, the shapes), as the reference's own include/dR_types.h lays them out.

Run in the build container, where /root/reference, the glib headers and the OpenCL headers exist: a small C
program that includes ONLY the reference's dR_types.h is compiled with gcc and prints offsetof() of every field
named below.  The output is a list of numbers (data); no text of the reference's header is kept.
tests/c_caller.c checks this library's include/dR_types.h against them with _Static_assert.
"""
import os
import subprocess
import sys
import tempfile

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
INC = ["-I" + os.path.join(REF, "include"), "-I/opt/conda/include/glib-2.0", "-I/opt/conda/lib/glib-2.0/include", "-I/usr/include"]

FIELDS = {
    "dR_Shape2": ["s0", "s1"],
    "dR_Shape3": ["s0", "s1", "s2"],
    "dR_Shape4": ["s0", "s1", "s2", "s3"],
    "dR_Config": ["silent", "profilingGPU", "profilingCPU", "debugInfo", "totalNodeCPUTime", "convLocalWorkSizeWindow", "modelPath"],
    "dR_ClConfig": ["clContext", "clPlatformId", "clCommandQueue", "clProgram", "clDeviceType", "clDeviceNumber", "clPlatformName",
                    "clKernelPath", "clDeviceId", "clNumDevices", "clDeviceIds", "clDeviceName", "clError", "clEventObject", "clEvent",
                    "forceRecompile", "totalKernelGPUTime", "queueKernelGPUTime", "maxTotalKernelGPUTime", "sumTotalKernelGPUTime",
                    "clInfo", "fastRelaxedMath", "build_status", "cleanupDone", "configH", "memConsumptionGPU"],
    "dR_Graph": ["prepared", "swapBuffer1", "swapBuffer2", "config", "clConfig", "feed_layers", "output_layers", "streamBufferHandlers",
                 "number_of_layers", "maxBufferSize", "hostDebugBuffer", "scheduledLayers", "allNodes", "debugLayer"],
    "dR_Node": ["oshape", "layerID", "previous_layers", "next_layers", "clKernel", "outputBuf", "layer", "type", "propagated", "output",
                "queued", "compute", "schedule", "propagateShape", "getRequiredOutputBufferSize", "createKernel", "allocateBuffers",
                "fillBuffers", "cleanupBuffers", "cleanupLayer", "printLayer", "serializeNode", "parseAppendNode", "generateKernel",
                "createKernelName", "setVariables"],
    "dR_MemoryHandler": ["outputFor", "size", "numberOfDependencies", "bufptr", "buf", "outputBuf", "regionOfInterest",
                         "useIndexBufferForRoI", "indexBuffer", "index", "roiOrigin"],
    "dR_ListElement": ["next", "previous", "element"],
    "dR_List": ["first", "last", "length", "iterator"],
}

src = ['#include <stdio.h>', '#include <stddef.h>', '#include "dR_types.h"', 'int main(void) {']
for s, fields in FIELDS.items():
    src.append('  printf("#define REF_SIZEOF_%s %%zu\\n", sizeof(%s));' % (s, s))
    for f in fields:
        src.append('  printf("#define REF_OFFSETOF_%s_%s %%zu\\n", offsetof(%s, %s));' % (s, f, s, f))
src += ['  return 0;', '}']
with tempfile.TemporaryDirectory() as tmp:
    c, exe = os.path.join(tmp, "offsets.c"), os.path.join(tmp, "offsets")
    open(c, "w").write("\n".join(src) + "\n")
    subprocess.run(["gcc", "-std=gnu99", "-w"] + INC + [c, "-o", exe], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
with open(os.path.join(HERE, "ref_struct_offsets.h"), "w") as f:
    f.write("/* Sizes and field offsets of the reference's include/dR_types.h on x86-64 Linux (gcc, glib 2, OpenCL headers),\n"
            " * written by tests/golden/make_struct_offsets.py.  Data only. */\n" + out)
print("%d lines written" % out.count("\n"))
