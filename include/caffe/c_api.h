/*
 * C ABI of the Mini-Caffe forward path (MI355X / HIP build of libcaffe.so).
 *
 * Binary-compatible with the reference's include/caffe/c_api.h:18-162, which
 * its ctypes binding (python/minicaffe/base.py:40-47), its JNI shim
 * (src/jni/jni.c:29-193) and tests/run_net.c bind against: same names, same
 * argument order and types, same conventions.
 *
 * Conventions
 *   - Handles are opaque pointers owned by the library.  A BlobHandle obtained
 *     from a net stays valid until CaffeNetDestroy.
 *   - Functions returning int give 0 on success and -1 on failure; the message
 *     is then available from CaffeGetLastError() on the same thread.
 *     The CaffeBlob{Num,Channels,Height,Width,Count} getters return the value.
 *   - Arrays handed out through int** / const char*** / BlobHandle** point into
 *     per-thread storage that the next call on that thread may overwrite.
 *   - CaffeBlobData returns the HOST mirror of the blob and marks it as the
 *     valid copy: write inputs through it before CaffeNetForward, read outputs
 *     through it afterwards (device results are copied back on first access).
 *     The pointer is invalidated by a reshape that grows the blob.
 *   - One net per thread; CaffeSetMode applies to the calling thread only.
 *     CaffeSetMode(1, device) selects the HIP path.  This build holds no CPU
 *     arithmetic: in mode 0 nets can be created, reshaped and inspected, but
 *     CaffeNetForward fails with an explanatory error.
 */
#ifndef CAFFE_C_API_H_
#define CAFFE_C_API_H_

#define CAFFE_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

typedef float real_t;
typedef void* BlobHandle;
typedef void* NetHandle;

/* ---- thread state and errors (reference c_api.h:139-162) -------------------- */

/* 1 when a HIP device can be used, 0 otherwise. */
CAFFE_API int CaffeGPUAvailable();
/* mode: 1 = GPU (HIP), 0 = CPU; device: HIP device id (-1 / ignored for CPU). */
CAFFE_API int CaffeSetMode(int mode, int device);
/* Message of the last failed call on this thread. */
CAFFE_API const char* CaffeGetLastError();
/* Return unused host and device blocks of this thread's pool to the system. */
CAFFE_API int CaffeMemoryPoolClear();

/* ---- Blob (reference c_api.h:24-44) ------------------------------------------ */

CAFFE_API int CaffeBlobNum(BlobHandle blob);
CAFFE_API int CaffeBlobChannels(BlobHandle blob);
CAFFE_API int CaffeBlobHeight(BlobHandle blob);
CAFFE_API int CaffeBlobWidth(BlobHandle blob);
CAFFE_API int CaffeBlobCount(BlobHandle blob);
CAFFE_API real_t* CaffeBlobData(BlobHandle blob);
/* New shape of shape_size axes; may move the data pointer. */
CAFFE_API int CaffeBlobReshape(BlobHandle blob, int shape_size, int* shape);
/* *shape points at shape_size ints in per-thread storage. */
CAFFE_API int CaffeBlobShape(BlobHandle blob, int* shape_size, int** shape);

/* ---- Net (reference c_api.h:46-116) ------------------------------------------ */

/* net_path: text prototxt; model_path: binary caffemodel. */
CAFFE_API int CaffeNetCreate(const char* net_path, const char* model_path, NetHandle* net);
/* net_buffer: text prototxt bytes; model_buffer: binary caffemodel bytes. */
CAFFE_API int CaffeNetCreateFromBuffer(const char* net_buffer, int nb_len,
                                       const char* model_buffer, int mb_len, NetHandle* net);
CAFFE_API int CaffeNetDestroy(NetHandle net);
/* Keep an internal blob readable after Forward (its memory is not recycled). */
CAFFE_API int CaffeNetMarkOutput(NetHandle net, const char* name);
/* Fill the input blobs first.  Equivalent to Net::Forward(true). */
CAFFE_API int CaffeNetForward(NetHandle net);
CAFFE_API int CaffeNetGetBlob(NetHandle net, const char* name, BlobHandle* blob);
/* All internal blobs, in creation order. */
CAFFE_API int CaffeNetListBlob(NetHandle net, int* n, const char*** names, BlobHandle** blobs);
/* All layer parameter blobs; names are "<layer>_<index>" unless the prototxt names them. */
CAFFE_API int CaffeNetListParam(NetHandle net, int* n, const char*** names,
                                BlobHandle** params);

/* ---- Profiler (reference c_api.h:118-137); not for multi-threaded use --------- */

CAFFE_API int CaffeProfilerEnable();
CAFFE_API int CaffeProfilerDisable();
CAFFE_API int CaffeProfilerScopeStart(const char* name);
CAFFE_API int CaffeProfilerScopeEnd();
/* Write chrome://tracing JSON to the file fn. */
CAFFE_API int CaffeProfilerDump(const char* fn);

#ifdef __cplusplus
}
#endif

#endif /* CAFFE_C_API_H_ */
