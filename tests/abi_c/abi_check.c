/* Plain C99 client of the library: proves that include/d3d_spconv.h is a C header and that the exported entry
 * points can be driven without Python or C++.  No kernel is launched: create / clone / serialize / shape inference /
 * error reporting only.  Usage: abi_check <path to libdeploy3d_amd.so>; exit code 0 = every check passed. */
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>

#include "d3d_spconv.h"

#define CHECK(cond)                                                   \
  do {                                                                \
    if (!(cond)) {                                                    \
      fprintf(stderr, "abi_check: %s failed (line %d)\n", #cond, __LINE__); \
      return 1;                                                       \
    }                                                                 \
  } while (0)

typedef int32_t (*create_fn)(const char*, const char*, const void*, size_t, d3d_plugin**);
typedef int32_t (*clone_fn)(const d3d_plugin*, d3d_plugin**);
typedef void (*destroy_fn)(d3d_plugin*);
typedef size_t (*size_fn)(const d3d_plugin*);
typedef int32_t (*serialize_fn)(const d3d_plugin*, void*, size_t);
typedef int32_t (*num_outputs_fn)(const d3d_plugin*);
typedef int32_t (*dims_fn)(const d3d_plugin*, int32_t, const d3d_tensor_desc*, int32_t, d3d_tensor_desc*);
typedef const char* (*str_fn)(void);
typedef const char* (*type_fn)(const d3d_plugin*);
typedef int32_t (*count_fn)(void);
typedef const char* (*name_fn)(int32_t);
typedef int32_t (*link_fn)(d3d_plugin*, d3d_plugin*);
typedef int32_t (*option_fn)(d3d_plugin*, int32_t, int64_t);
typedef int32_t (*sched_create_fn)(int32_t, d3d_schedule**);
typedef int32_t (*sched_add_fn)(d3d_schedule*, d3d_plugin*, const d3d_tensor_desc*, int32_t, const d3d_tensor_desc*,
                                int32_t, const void* const*, void* const*, void*, size_t, int32_t, const int32_t*,
                                int32_t);
typedef int32_t (*sched_size_fn)(const d3d_schedule*);
typedef void (*sched_destroy_fn)(d3d_schedule*);

int main(int argc, char** argv) {
  CHECK(argc == 2);
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    fprintf(stderr, "abi_check: %s\n", dlerror());
    return 1;
  }
  create_fn create = (create_fn)dlsym(lib, "d3d_create");
  clone_fn clone = (clone_fn)dlsym(lib, "d3d_clone");
  destroy_fn destroy = (destroy_fn)dlsym(lib, "d3d_destroy");
  size_fn ser_size = (size_fn)dlsym(lib, "d3d_serialize_size");
  serialize_fn serialize = (serialize_fn)dlsym(lib, "d3d_serialize");
  num_outputs_fn num_outputs = (num_outputs_fn)dlsym(lib, "d3d_num_outputs");
  dims_fn output_dims = (dims_fn)dlsym(lib, "d3d_output_dims");
  str_fn last_error = (str_fn)dlsym(lib, "d3d_last_error");
  type_fn plugin_type = (type_fn)dlsym(lib, "d3d_plugin_type");
  count_fn num_ops = (count_fn)dlsym(lib, "d3d_num_ops");
  name_fn op_name = (name_fn)dlsym(lib, "d3d_op_name");
  link_fn link_rulebook = (link_fn)dlsym(lib, "d3d_link_rulebook");
  option_fn set_option = (option_fn)dlsym(lib, "d3d_set_option");
  sched_create_fn sched_create = (sched_create_fn)dlsym(lib, "d3d_schedule_create");
  sched_add_fn sched_add = (sched_add_fn)dlsym(lib, "d3d_schedule_add");
  sched_size_fn sched_size = (sched_size_fn)dlsym(lib, "d3d_schedule_size");
  sched_destroy_fn sched_destroy = (sched_destroy_fn)dlsym(lib, "d3d_schedule_destroy");
  CHECK(create && clone && destroy && ser_size && serialize && num_outputs && output_dims && last_error &&
        plugin_type && num_ops && op_name && link_rulebook && set_option && sched_create && sched_add &&
        sched_size && sched_destroy);

  CHECK(num_ops() >= 5);
  CHECK(strcmp(op_name(2), "SPConvIdx3d") == 0);

  /* SPConvIdxPluginParam<3>: 5 x int32[3], int32 maxNumActOut, u8 subM, u8 transpose = 66 bytes */
  unsigned char blob[66];
  const int32_t fields[16] = {3, 3, 3, 2, 2, 2, 1, 1, 1, 1, 1, 1, 0, 0, 0, 5000};
  memcpy(blob, fields, 64);
  blob[64] = 0;
  blob[65] = 0;
  d3d_plugin* p = NULL;
  CHECK(create("SPConvIdx3d", "2.0", blob, sizeof(blob), &p) == D3D_OK && p);
  CHECK(strcmp(plugin_type(p), "SPConvIdx3d") == 0);
  CHECK(num_outputs(p) == 5);
  CHECK(ser_size(p) == sizeof(blob));
  unsigned char back[66];
  CHECK(serialize(p, back, sizeof(back)) == D3D_OK && memcmp(back, blob, sizeof(blob)) == 0);

  d3d_tensor_desc in[3];
  memset(in, 0, sizeof(in));
  in[0].dtype = D3D_INT32; in[0].nb_dims = 2; in[0].dims[0] = 20000; in[0].dims[1] = 4;
  in[1].dtype = D3D_INT32; in[1].nb_dims = 1; in[1].dims[0] = 1;
  in[2].dtype = D3D_INT32; in[2].nb_dims = 5;
  in[2].dims[0] = 2; in[2].dims[1] = 0; in[2].dims[2] = 41; in[2].dims[3] = 1440; in[2].dims[4] = 1440;
  d3d_tensor_desc out;
  CHECK(output_dims(p, 0, in, 3, &out) == D3D_OK && out.nb_dims == 2 && out.dims[0] == 3 &&
        out.dims[1] == 27 * (20000 + 128));
  CHECK(output_dims(p, 4, in, 3, &out) == D3D_OK && out.nb_dims == 5 && out.dims[2] == 21 && out.dims[3] == 720);

  d3d_plugin* q = NULL;
  CHECK(clone(p, &q) == D3D_OK && q && ser_size(q) == sizeof(blob));

  /* SPConvMMPluginParam: 4 x int32, 3 x u8, then fp32 W[kVol*Cin*Cout] (1x1x1 kernel, 2 -> 2 channels) */
  unsigned char mm_blob[19 + 16];
  const int32_t mm_fields[4] = {1, 2, 2, 5000};
  const float mm_w[4] = {1.f, 0.f, 0.f, 1.f};
  memcpy(mm_blob, mm_fields, 16);
  mm_blob[16] = 0; mm_blob[17] = 0; mm_blob[18] = 0;
  memcpy(mm_blob + 19, mm_w, 16);
  d3d_plugin* mm = NULL;
  CHECK(create("SPConvMM", "2.0", mm_blob, sizeof(mm_blob), &mm) == D3D_OK && mm);
  /* linking checks its operands before it touches the device */
  CHECK(link_rulebook(p, q) == D3D_ERR_BAD_ARG);           /* first handle is not a convolution */
  CHECK(link_rulebook(mm, mm) == D3D_ERR_BAD_ARG);         /* second handle is not a rulebook operator */
  CHECK(link_rulebook(mm, p) == D3D_ERR_BAD_ARG);          /* kernel volume 1 against 27 */
  CHECK(link_rulebook(mm, NULL) == D3D_OK);                /* removing a link that is not there */
  CHECK(set_option(mm, D3D_OPT_PERSISTENT_INDEX, 1) == D3D_ERR_UNSUPPORTED && strlen(last_error()) > 0);
  CHECK(set_option(p, 12345, 1) == D3D_ERR_UNSUPPORTED);
  CHECK(set_option(NULL, D3D_OPT_PERSISTENT_INDEX, 1) == D3D_ERR_BAD_ARG);
  /* a one-lane schedule is pure bookkeeping (no stream, no event): steps are copied, bad steps refused */
  d3d_schedule* sched = NULL;
  CHECK(sched_create(0, &sched) == D3D_ERR_BAD_ARG && sched == NULL);
  CHECK(sched_create(1, &sched) == D3D_OK && sched && sched_size(sched) == 0);
  {
    d3d_tensor_desc outs[5];
    const void* in_ptrs[3] = {NULL, NULL, NULL};
    void* out_ptrs[5] = {NULL, NULL, NULL, NULL, NULL};
    const int32_t first = 0, self = 2;   /* the third step would be step 2 */
    for (int i = 0; i < 5; ++i) CHECK(output_dims(p, i, in, 3, &outs[i]) == D3D_OK);
    CHECK(sched_add(sched, p, in, 3, outs, 5, in_ptrs, out_ptrs, NULL, 0, 0, NULL, 0) == 0);
    CHECK(sched_add(sched, q, in, 3, outs, 5, in_ptrs, out_ptrs, NULL, 0, 0, &first, 1) == 1);
    CHECK(sched_add(sched, p, in, 3, outs, 4, in_ptrs, out_ptrs, NULL, 0, 0, NULL, 0) == D3D_ERR_BAD_ARG);
    CHECK(sched_add(sched, p, in, 3, outs, 5, in_ptrs, out_ptrs, NULL, 0, 1, NULL, 0) == D3D_ERR_BAD_ARG);
    CHECK(sched_add(sched, p, in, 3, outs, 5, in_ptrs, out_ptrs, NULL, 0, 0, &self, 1) == D3D_ERR_BAD_ARG);
    CHECK(sched_size(sched) == 2);
  }
  sched_destroy(sched);
  sched_destroy(NULL);
  destroy(mm);
  destroy(q);
  destroy(p);

  /* errors come back as status codes with a message, never as exceptions */
  p = NULL;
  CHECK(create("SPConvIdx3d", "2.0", blob, 10, &p) == D3D_ERR_BAD_BLOB && p == NULL && strlen(last_error()) > 0);
  CHECK(create("NoSuchOp", "2.0", blob, sizeof(blob), &p) == D3D_ERR_UNKNOWN_OP);
  dlclose(lib);
  printf("abi_check ok\n");
  return 0;
}
