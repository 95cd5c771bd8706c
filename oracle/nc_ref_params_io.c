/* TEST INFRASTRUCTURE (CPU checker): parameter files, libnc.h:524-536, 580.
   libnc's own file layout is not published with the header, so this is the layout the
   product library defines (little-endian: "NCPF", u32 version 1, u32 config length, config;
   then per parameter u32 name length, name, u32 type, u32 n_dims, u64 dims[], elements in
   memory order), written here a second time against the public tensor API only, so that a
   file saved by one library and loaded by the other is a test of both.  Parity with libnc's
   files: unpinned (no such file exists in the reference tree). */
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include "nc_ref_internal.h"

static void wr(FILE *f, const void *p, size_t n)
{
    if (n && fwrite(p, n, 1, f) != 1)
        nc_fatal("parameter file: write failed");
}

static size_t numel_of(const NCTensor *x, size_t *dims, int *nd)
{
    size_t n = 1;
    *nd = nc_tensor_get_dims(x, dims);
    for (int i = 0; i < *nd; i++)
        n *= dims[i];
    return n;
}

NCParam *nc_find_param(NCParamList *pl, const char *name)
{
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next)
        if (!strcmp(((NCParam *)el)->name, name))
            return (NCParam *)el;
    return NULL;
}

void nc_save_param_header(FILE *f, const char *config)
{
    uint32_t v = 1, n = config ? (uint32_t)strlen(config) : 0;
    wr(f, "NCPF", 4); wr(f, &v, 4); wr(f, &n, 4); wr(f, config, n);
}

char *nc_load_param_header(FILE *f)
{
    char magic[4];
    uint32_t v, n;
    if (fread(magic, 4, 1, f) != 1 || memcmp(magic, "NCPF", 4) || fread(&v, 4, 1, f) != 1 || v != 1 ||
        fread(&n, 4, 1, f) != 1 || n > (1u << 20))
        return NULL;
    char *cfg = nc_malloc(n + 1);
    if (n && fread(cfg, n, 1, f) != 1) {
        nc_free(cfg);
        return NULL;
    }
    cfg[n] = 0;
    return cfg;
}

void nc_save_param(FILE *f, const NCTensor *v1, const char *name)
{
    NCTensor *h = nc_tensor_to_cpu_device(nc_dup_tensor(v1));
    size_t dims[NC_N_DIMS_MAX], stride;
    int nd;
    size_t n = numel_of(h, dims, &nd);
    uint32_t nl = (uint32_t)strlen(name), type = (uint32_t)nc_tensor_get_item_type(h), ndu = (uint32_t)nd;
    wr(f, &nl, 4); wr(f, name, nl); wr(f, &type, 4); wr(f, &ndu, 4);
    for (int i = 0; i < nd; i++) {
        uint64_t d = dims[i];
        wr(f, &d, 8);
    }
    wr(f, nc_tensor_get_ptr(h, &stride), n * nc_type_size(nc_tensor_get_item_type(h)));
    nc_free_tensor(h);
}

/* bytes between the read position and the end of the file */
static uint64_t bytes_left(FILE *f)
{
    long pos = ftell(f), end;
    if (pos < 0 || fseek(f, 0, SEEK_END))
        nc_fatal("parameter file: not seekable");
    end = ftell(f);
    if (end < pos || fseek(f, pos, SEEK_SET))
        nc_fatal("parameter file: not seekable");
    return (uint64_t)(end - pos);
}

NCTensor *nc_load_param(NCContext *m, FILE *f, char *name, size_t name_size)
{
    uint32_t nl, type, nd;
    size_t dims[NC_N_DIMS_MAX], n = 1, stride;
    uint64_t room;
    if (fread(&nl, 4, 1, f) != 1)
        return NULL;
    if ((size_t)nl >= name_size) /* in size_t: a 32-bit nl + 1 wraps for 0xffffffff */
        nc_fatal("parameter file: a name of %u bytes does not fit the caller's buffer", nl);
    if (nl && fread(name, nl, 1, f) != 1)
        nc_fatal("parameter file: truncated record");
    name[nl] = 0;
    if (fread(&type, 4, 1, f) != 1 || fread(&nd, 4, 1, f) != 1)
        nc_fatal("parameter file: truncated record '%s'", name);
    if (nd > NC_N_DIMS_MAX || type >= NC_TYPE_COUNT) /* nd = 0: a scalar */
        nc_fatal("parameter file: bad record '%s' (type %u, %u dimensions)", name, type, nd);
    room = bytes_left(f);
    if (room < (uint64_t)nd * 8)
        nc_fatal("parameter file: truncated record '%s'", name);
    room = (room - (uint64_t)nd * 8) / nc_type_size((NCTypeEnum)type);
    for (uint32_t i = 0; i < nd; i++) {
        uint64_t d;
        if (fread(&d, 8, 1, f) != 1)
            nc_fatal("parameter file: truncated record '%s'", name);
        if (d == 0 || d > room / n)
            nc_fatal("parameter file: record '%s' claims more elements than the file holds", name);
        dims[i] = (size_t)d;
        n *= dims[i];
    }
    if (room < n)
        nc_fatal("parameter file: truncated record '%s'", name);
    NCTensor *h = nc_new_tensor(nc_new_cpu_device(m), (NCTypeEnum)type, (int)nd, dims);
    size_t bytes = n * nc_type_size((NCTypeEnum)type);
    if (bytes && fread(nc_tensor_get_ptr(h, &stride), bytes, 1, f) != 1)
        nc_fatal("parameter file: truncated record '%s'", name);
    return h;
}

void nc_update_param(NCParamList *pl, const char *name, const NCTensor *v)
{
    NCParam *p = nc_find_param(pl, name);
    size_t da[NC_N_DIMS_MAX], db[NC_N_DIMS_MAX];
    int na, nb;
    if (!p)
        nc_fatal("nc_update_param: no parameter named '%s'", name);
    NCTensor *dst = *p->pval;
    numel_of(dst, da, &na);
    numel_of(v, db, &nb);
    if (na != nb || memcmp(da, db, sizeof(size_t) * na) || nc_tensor_get_item_type(dst) != nc_tensor_get_item_type(v))
        nc_fatal("nc_update_param: '%s' has another shape or type", name);
    NCTensor *src = nc_tensor_to_device(nc_dup_tensor(v), nc_get_tensor_device(dst));
    nc_tensor_copy(dst, src);
    nc_free_tensor(src);
}

void nc_save_coefs(NCParamList *pl, const char *filename)
{
    FILE *f = fopen(filename, "wb");
    if (!f)
        nc_fatal("nc_save_coefs: cannot write '%s'", filename);
    nc_save_param_header(f, "");
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next)
        nc_save_param(f, *((NCParam *)el)->pval, ((NCParam *)el)->name);
    if (fclose(f))
        nc_fatal("nc_save_coefs: write to '%s' failed", filename);
}

void nc_load_coefs(NCParamList *pl, const char *filename)
{
    FILE *f = fopen(filename, "rb");
    char name[256], *cfg;
    NCTensor *h;
    if (!f)
        nc_fatal("nc_load_coefs: cannot read '%s'", filename);
    cfg = nc_load_param_header(f);
    if (!cfg)
        nc_fatal("nc_load_coefs: '%s' is not a parameter file", filename);
    nc_free(cfg);
    while ((h = nc_load_param(pl->ctx, f, name, sizeof(name))) != NULL) {
        nc_update_param(pl, name, h);
        nc_free_tensor(h);
    }
    fclose(f);
}
