// Parameter files: nc_save_coefs / nc_load_coefs and the record-level calls under them
// (libnc.h:524-536, 580).  libnc's own file layout is not published with the header, so the
// layout is defined here: little-endian,
//   header  "NCPF" u32 version (1) u32 config_len, config bytes
//   record  u32 name_len, name bytes, u32 type (NCTypeEnum), u32 n_dims, u64 dims[n_dims],
//           the elements in memory order (dims[0] innermost)
// up to the end of the file.  Records are written from host copies of the tensors and read
// into host tensors; nc_load_coefs copies each record into the parameter of the same name
// on whatever device that parameter lives (shape and type must match; names the list does
// not hold are an error, parameters the file does not hold keep their values).
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include "nc_hip_internal.h"

namespace {

const char MAGIC[4] = { 'N', 'C', 'P', 'F' };

void put_u32(FILE *f, uint32_t v) { if (fwrite(&v, 4, 1, f) != 1) nc_fatal("parameter file: write failed"); }
void put_u64(FILE *f, uint64_t v) { if (fwrite(&v, 8, 1, f) != 1) nc_fatal("parameter file: write failed"); }
bool get_u32(FILE *f, uint32_t *v) { return fread(v, 4, 1, f) == 1; }
bool get_u64(FILE *f, uint64_t *v) { return fread(v, 8, 1, f) == 1; }

} // namespace

extern "C" NCParam *nc_find_param(NCParamList *pl, const char *name) // libnc.h:524
{
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next) {
        NCParam *p = (NCParam *)el;
        if (!strcmp(p->name, name)) return p;
    }
    return nullptr;
}

extern "C" void nc_save_param_header(FILE *f, const char *config) // libnc.h:528
{
    if (fwrite(MAGIC, 4, 1, f) != 1) nc_fatal("parameter file: write failed");
    put_u32(f, 1);
    uint32_t n = config ? (uint32_t)strlen(config) : 0;
    put_u32(f, n);
    if (n && fwrite(config, n, 1, f) != 1) nc_fatal("parameter file: write failed");
}

extern "C" char *nc_load_param_header(FILE *f) // libnc.h:533: NULL on error, nc_free() the result
{
    char magic[4];
    uint32_t version, n;
    if (fread(magic, 4, 1, f) != 1 || memcmp(magic, MAGIC, 4) || !get_u32(f, &version) || version != 1 ||
        !get_u32(f, &n) || n > (1u << 20))
        return nullptr;
    char *cfg = (char *)nc_malloc(n + 1);
    if (n && fread(cfg, n, 1, f) != 1) { nc_free(cfg); return nullptr; }
    cfg[n] = 0;
    return cfg;
}

extern "C" void nc_save_param(FILE *f, const NCTensor *v1, const char *name) // libnc.h:529
{
    NCTensor *h = nc_tensor_to_cpu_device(nc_dup_tensor(v1)); // contiguous host copy
    uint32_t nl = (uint32_t)strlen(name);
    put_u32(f, nl);
    if (nl && fwrite(name, nl, 1, f) != 1) nc_fatal("parameter file: write failed");
    put_u32(f, (uint32_t)h->type);
    put_u32(f, (uint32_t)h->n_dims);
    for (int i = 0; i < h->n_dims; i++) put_u64(f, (uint64_t)h->dims[i]);
    size_t bytes = nc_numel(h) * nc_type_size(h->type);
    if (bytes && fwrite(nc_data(h), bytes, 1, f) != 1) nc_fatal("parameter file: write failed");
    nc_free_tensor(h);
}

// libnc.h:535: the next record as a host tensor, NULL at the end of the file
extern "C" NCTensor *nc_load_param(NCContext *m, FILE *f, char *name, size_t name_size)
{
    uint32_t nl, type, nd;
    if (!get_u32(f, &nl)) return nullptr;
    // (compared as size_t: nl + 1 wraps to 0 for a name length of 0xffffffff)
    if (name_size == 0 || (size_t)nl >= name_size)
        nc_fatal("parameter file: a name of %u bytes does not fit the caller's buffer", nl);
    if (nl && fread(name, nl, 1, f) != 1) nc_fatal("parameter file: truncated record");
    name[nl] = 0;
    if (!get_u32(f, &type) || !get_u32(f, &nd)) nc_fatal("parameter file: truncated record '%s'", name);
    // (no dimensions: a scalar parameter, one element)
    if (nd > NC_N_DIMS_MAX || type >= (uint32_t)NC_TYPE_COUNT)
        nc_fatal("parameter file: bad record '%s' (type %u, %u dimensions)", name, type, nd);
    size_t dims[NC_N_DIMS_MAX];
    // what the file still holds bounds the record: checked before anything is allocated
    const long here = ftell(f);
    if (here < 0 || fseek(f, 0, SEEK_END) != 0) nc_fatal("parameter file: not seekable");
    const long end = ftell(f);
    if (end < here || fseek(f, here, SEEK_SET) != 0) nc_fatal("parameter file: not seekable");
    const uint64_t left = (uint64_t)(end - here), esz = nc_type_size((NCTypeEnum)type);
    if (left < 8ull * nd) nc_fatal("parameter file: truncated record '%s'", name);
    uint64_t budget = (left - 8ull * nd) / esz, count = 1; // elements the rest of the file can hold
    for (uint32_t i = 0; i < nd; i++) {
        uint64_t d;
        if (!get_u64(f, &d)) nc_fatal("parameter file: truncated record '%s'", name);
        if (d == 0 || d > budget / count)
            nc_fatal("parameter file: record '%s' claims more elements than the file holds", name);
        count *= d;
        dims[i] = (size_t)d;
    }
    if (budget < count) nc_fatal("parameter file: truncated record '%s'", name);
    NCTensor *h = nc_new_tensor(nc_new_cpu_device(m), (NCTypeEnum)type, (int)nd, dims);
    size_t bytes = nc_numel(h) * nc_type_size(h->type);
    if (bytes && fread(nc_data(h), bytes, 1, f) != 1) nc_fatal("parameter file: truncated record '%s'", name);
    return h;
}

extern "C" void nc_update_param(NCParamList *pl, const char *name, const NCTensor *v) // libnc.h:580
{
    NCParam *p = nc_find_param(pl, name);
    if (!p) nc_fatal("nc_update_param: no parameter named '%s'", name);
    NCTensor *dst = *p->pval;
    if (dst->type != v->type || dst->n_dims != v->n_dims || memcmp(dst->dims, v->dims, sizeof(size_t) * v->n_dims))
        nc_fatal("nc_update_param: '%s' has another shape or type", name);
    NCTensor *src = nc_tensor_to_device(nc_dup_tensor(v), nc_get_tensor_device(dst));
    nc_tensor_copy(dst, src);
    nc_free_tensor(src);
}

extern "C" void nc_save_coefs(NCParamList *pl, const char *filename) // libnc.h:530
{
    FILE *f = fopen(filename, "wb");
    if (!f) nc_fatal("nc_save_coefs: cannot write '%s'", filename);
    nc_save_param_header(f, "");
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next) {
        NCParam *p = (NCParam *)el;
        nc_save_param(f, *p->pval, p->name);
    }
    if (fclose(f)) nc_fatal("nc_save_coefs: write to '%s' failed", filename);
}

extern "C" void nc_load_coefs(NCParamList *pl, const char *filename) // libnc.h:536
{
    FILE *f = fopen(filename, "rb");
    if (!f) nc_fatal("nc_load_coefs: cannot read '%s'", filename);
    char *cfg = nc_load_param_header(f);
    if (!cfg) nc_fatal("nc_load_coefs: '%s' is not a parameter file", filename);
    nc_free(cfg);
    char name[256];
    for (;;) {
        NCTensor *h = nc_load_param(pl->ctx, f, name, sizeof(name));
        if (!h) break;
        nc_update_param(pl, name, h);
        nc_free_tensor(h);
    }
    fclose(f);
}
