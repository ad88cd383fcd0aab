/* STAND-IN, for syntax checking only.  This image has no Erlang/OTP, so nx_amd/elixir/c_src/hipnx_nif.c
 * cannot be compiled against the real <erl_nif.h>.  This header declares -- from the public erl_nif
 * documentation, declarations only, nothing is implemented -- exactly the types, constants and functions
 * the shim uses, so that `gcc -fsyntax-only` can prove their spelling and arity.  It proves nothing about
 * behaviour and is never linked or shipped. */
#ifndef ERL_NIF_STANDIN_H
#define ERL_NIF_STANDIN_H
#include <stddef.h>
#include <stdint.h>

typedef uint64_t ERL_NIF_TERM;
typedef int64_t ErlNifSInt64;
typedef uint64_t ErlNifUInt64;
typedef struct enif_environment_t ErlNifEnv;
typedef struct enif_resource_type_t ErlNifResourceType;
typedef struct {
  size_t size;
  unsigned char *data;
  void *ref_bin;
  void *spare_[2];
} ErlNifBinary;
typedef void ErlNifResourceDtor(ErlNifEnv *, void *);
typedef enum { ERL_NIF_RT_CREATE = 1, ERL_NIF_RT_TAKEOVER = 2 } ErlNifResourceFlags;
typedef enum { ERL_NIF_LATIN1 = 1 } ErlNifCharEncoding;
#define ERL_NIF_DIRTY_JOB_CPU_BOUND 1
#define ERL_NIF_DIRTY_JOB_IO_BOUND 2
typedef struct {
  const char *name;
  unsigned arity;
  ERL_NIF_TERM (*fptr)(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]);
  unsigned flags;
} ErlNifFunc;
typedef struct {
  int major, minor;
  const char *name;
  int num_of_funcs;
  ErlNifFunc *funcs;
  int (*load)(ErlNifEnv *, void **priv_data, ERL_NIF_TERM load_info);
  int (*reload)(ErlNifEnv *, void **priv_data, ERL_NIF_TERM load_info);
  int (*upgrade)(ErlNifEnv *, void **priv_data, void **old_priv_data, ERL_NIF_TERM load_info);
  void (*unload)(ErlNifEnv *, void *priv_data);
} ErlNifEntry;
#define ERL_NIF_INIT(NAME, FUNCS, LOAD, RELOAD, UPGRADE, UNLOAD)                                   \
  ErlNifEntry *nif_init(void) {                                                                    \
    static ErlNifEntry entry = {2, 16, #NAME, sizeof(FUNCS) / sizeof(*FUNCS), FUNCS, LOAD, RELOAD, UPGRADE, UNLOAD}; \
    return &entry;                                                                                 \
  }

ERL_NIF_TERM enif_make_badarg(ErlNifEnv *env);
ERL_NIF_TERM enif_make_atom(ErlNifEnv *env, const char *name);
ERL_NIF_TERM enif_make_tuple(ErlNifEnv *env, unsigned cnt, ...);
#define enif_make_tuple2(ENV, E1, E2) enif_make_tuple(ENV, 2, E1, E2)
#define enif_make_tuple3(ENV, E1, E2, E3) enif_make_tuple(ENV, 3, E1, E2, E3)
ERL_NIF_TERM enif_make_int(ErlNifEnv *env, int i);
ERL_NIF_TERM enif_make_uint(ErlNifEnv *env, unsigned i);
ERL_NIF_TERM enif_make_int64(ErlNifEnv *env, ErlNifSInt64 i);
ERL_NIF_TERM enif_make_uint64(ErlNifEnv *env, ErlNifUInt64 i);
ERL_NIF_TERM enif_make_string(ErlNifEnv *env, const char *string, ErlNifCharEncoding encoding);
unsigned char *enif_make_new_binary(ErlNifEnv *env, size_t size, ERL_NIF_TERM *termp);
int enif_get_int(ErlNifEnv *env, ERL_NIF_TERM term, int *ip);
int enif_get_uint(ErlNifEnv *env, ERL_NIF_TERM term, unsigned *ip);
int enif_get_int64(ErlNifEnv *env, ERL_NIF_TERM term, ErlNifSInt64 *ip);
int enif_get_uint64(ErlNifEnv *env, ERL_NIF_TERM term, ErlNifUInt64 *ip);
int enif_get_list_length(ErlNifEnv *env, ERL_NIF_TERM term, unsigned *len);
int enif_get_list_cell(ErlNifEnv *env, ERL_NIF_TERM list, ERL_NIF_TERM *head, ERL_NIF_TERM *tail);
int enif_inspect_binary(ErlNifEnv *env, ERL_NIF_TERM bin_term, ErlNifBinary *bin);
ErlNifResourceType *enif_open_resource_type(ErlNifEnv *env, const char *module_str, const char *name, ErlNifResourceDtor *dtor,
                                            ErlNifResourceFlags flags, ErlNifResourceFlags *tried);
void *enif_alloc_resource(ErlNifResourceType *type, size_t size);
void enif_release_resource(void *obj);
ERL_NIF_TERM enif_make_resource(ErlNifEnv *env, void *obj);
int enif_get_resource(ErlNifEnv *env, ERL_NIF_TERM term, ErlNifResourceType *type, void **objp);
#endif
