/*
 * dr_compat.h -- scalar and handle typedefs that let the deepRacin C graph API compile
 * without glib or an OpenCL SDK installed.
 *
 * The frozen public signatures (reference include/deepRACIN.h:18-279, include/dR_clwrap.h:20-49)
 * are spelled with glib scalars (gint, gfloat, gboolean, gchar ...) and OpenCL handle types
 * (cl_mem, cl_kernel ...).  This library links neither: the glib names are plain C typedefs with
 * glib's own widths, and the OpenCL handles are opaque pointers of the same size as the originals,
 * so every struct keeps the field offsets a caller compiled against the reference headers expects.
 *
 * A `cl_mem` produced by this library IS the HIP device address of the buffer (cast to the opaque
 * pointer type).  A HIP caller may therefore hand `*outptr[i]` straight to its own kernels.
 *
 * If the real headers were included first (glib.h / CL/cl.h) their definitions win.
 */
#ifndef DR_COMPAT_H
#define DR_COMPAT_H

#include <stddef.h>
#include <stdint.h>

/* ---- glib scalars -------------------------------------------------------------------------- */
#if !defined(__G_LIB_H__) && !defined(__G_TYPES_H__)
typedef char            gchar;
typedef int             gint;
typedef gint            gboolean;
typedef int32_t         gint32;
typedef int64_t         gint64;
typedef unsigned int    guint;
typedef long            glong;
typedef float           gfloat;
typedef double          gdouble;
typedef size_t          gsize;
typedef void*           gpointer;
#ifndef FALSE
#define FALSE (0)
#endif
#ifndef TRUE
#define TRUE (!FALSE)
#endif
#endif

/* ---- OpenCL scalars and opaque handles ----------------------------------------------------- */
#if !defined(__OPENCL_CL_H) && !defined(__CL_PLATFORM_H) && !defined(CL_VERSION_1_0)
typedef int32_t         cl_int;
typedef uint32_t        cl_uint;
typedef uint64_t        cl_ulong;
typedef float           cl_float;
typedef cl_int          cl_build_status;
typedef struct _cl_platform_id*   cl_platform_id;
typedef struct _cl_device_id*     cl_device_id;
typedef struct _cl_context*       cl_context;
typedef struct _cl_command_queue* cl_command_queue;
typedef struct _cl_mem*           cl_mem;
typedef struct _cl_program*       cl_program;
typedef struct _cl_kernel*        cl_kernel;
typedef struct _cl_event*         cl_event;
/* buffer-type argument of dR_createFloatBuffer; accepted and ignored (all HIP buffers are RW) */
#define CL_MEM_READ_WRITE   (1 << 0)
#define CL_MEM_WRITE_ONLY   (1 << 1)
#define CL_MEM_READ_ONLY    (1 << 2)
#define CL_DEVICE_TYPE_CPU  (1 << 1)
#define CL_DEVICE_TYPE_GPU  (1 << 2)
#endif

#endif /* DR_COMPAT_H */
