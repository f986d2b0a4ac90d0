/* A C99 consumer of the C ABI, in the spirit of the reference's tests/run_net.c:
 *
 *   run_net_c net.prototxt net.caffemodel
 *
 * Compiled as C (not C++) against include/caffe/c_api.h, so it also checks that the
 * header is valid C.  Walks the calls a C program makes: device selection, net from
 * files, input blob shape / reshape / data, forward, blob and parameter listing, the
 * -1 + CaffeGetLastError convention, net from memory buffers, destruction.
 * Prints one line per step and "run_net_c: ok" at the end; exits 1 on any failure. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <caffe/c_api.h>

static void must(int rc, const char* what) {
  if (rc != 0) {
    printf("%s failed: %s\n", what, CaffeGetLastError());
    exit(1);
  }
}

static char* slurp(const char* path, long* size) {
  FILE* f = fopen(path, "rb");
  char* buf;
  if (!f) {
    printf("cannot open %s\n", path);
    exit(1);
  }
  fseek(f, 0, SEEK_END);
  *size = ftell(f);
  fseek(f, 0, SEEK_SET);
  buf = (char*)malloc((size_t)*size + 1);
  if (fread(buf, 1, (size_t)*size, f) != (size_t)*size) {
    printf("short read on %s\n", path);
    exit(1);
  }
  buf[*size] = 0;
  fclose(f);
  return buf;
}

int main(int argc, char* argv[]) {
  NetHandle net = NULL, net2 = NULL;
  BlobHandle data = NULL, out = NULL;
  BlobHandle* blobs = NULL;
  const char** names = NULL;
  int* shape = NULL;
  int n = 0, i, count, axes = 0;
  long proto_size = 0, model_size = 0;
  char *proto, *model;
  real_t* p;
  double sum = 0.;
  if (argc != 3) {
    printf("usage: run_net_c net.prototxt net.caffemodel\n");
    return 1;
  }
  if (CaffeGPUAvailable()) must(CaffeSetMode(1, 0), "CaffeSetMode");
  must(CaffeNetCreate(argv[1], argv[2], &net), "CaffeNetCreate");
  must(CaffeNetGetBlob(net, "data", &data), "CaffeNetGetBlob(data)");
  must(CaffeBlobShape(data, &axes, &shape), "CaffeBlobShape");
  count = CaffeBlobCount(data);
  printf("data: %d axes, [%d, %d, %d, %d], %d values\n", axes, CaffeBlobNum(data), CaffeBlobChannels(data),
         CaffeBlobHeight(data), CaffeBlobWidth(data), count);
  if (count != CaffeBlobNum(data) * CaffeBlobChannels(data) * CaffeBlobHeight(data) * CaffeBlobWidth(data)) {
    printf("count does not match the extents\n");
    return 1;
  }
  {
    int same[4];
    same[0] = CaffeBlobNum(data);
    same[1] = CaffeBlobChannels(data);
    same[2] = CaffeBlobHeight(data);
    same[3] = CaffeBlobWidth(data);
    must(CaffeBlobReshape(data, 4, same), "CaffeBlobReshape");
  }
  p = CaffeBlobData(data);
  for (i = 0; i < count; ++i) p[i] = (real_t)((i * 37 % 101) / 50.0 - 1.0);
  must(CaffeNetForward(net), "CaffeNetForward");
  must(CaffeNetListBlob(net, &n, &names, &blobs), "CaffeNetListBlob");
  printf("%d blobs\n", n);
  for (i = 0; i < n; ++i)
    printf("  %s: [%d, %d, %d, %d]\n", names[i], CaffeBlobNum(blobs[i]), CaffeBlobChannels(blobs[i]),
           CaffeBlobHeight(blobs[i]), CaffeBlobWidth(blobs[i]));
  out = blobs[n - 1];
  p = CaffeBlobData(out);
  for (i = 0; i < CaffeBlobCount(out); ++i) sum += p[i];
  printf("sum of the last blob: %.6f, first value: %.8f\n", sum, (double)p[0]);
  must(CaffeNetListParam(net, &n, &names, &blobs), "CaffeNetListParam");
  printf("%d parameter blobs, first: %s\n", n, n > 0 ? names[0] : "-");
  must(CaffeNetDestroy(net), "CaffeNetDestroy");

  if (CaffeNetCreate("no-such-prototxt", "no-such-caffemodel", &net2) != -1 || strlen(CaffeGetLastError()) == 0) {
    printf("missing files must give -1 and a message\n");
    return 1;
  }
  printf("expected error: %s\n", CaffeGetLastError());

  proto = slurp(argv[1], &proto_size);
  model = slurp(argv[2], &model_size);
  must(CaffeNetCreateFromBuffer(proto, (int)proto_size, model, (int)model_size, &net2), "CaffeNetCreateFromBuffer");
  must(CaffeNetDestroy(net2), "CaffeNetDestroy");
  must(CaffeMemoryPoolClear(), "CaffeMemoryPoolClear");
  free(proto);
  free(model);
  printf("run_net_c: ok\n");
  return 0;
}
