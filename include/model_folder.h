/* model_folder.h - NanoSeedLM model folders (safetensors shards + model.safetensors.index.json) and expert bank files read
 * into the prepacked HBM layout.  Mirrors the reference's reader: nslm/model_st.h:1-86 (logical tensors and their
 * streams), nslm/lib_model_st.c:36-300 (stream lengths, entry grouping, affine group rules, config.json's quantization
 * block), nslm/lib_format.c:50-140 (safetensors header), nslm/lib_moe.c:92-107 (.blk / .blk4 bank -> streams).
 * C99 + POSIX; the files are mapped read-only and streams point into the mappings. */
#ifndef NSLM_MODEL_FOLDER_H
#define NSLM_MODEL_FOLDER_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* encodings = MF_* of the kernels (nslm/model_st.h:31-34) */
enum { NSF_BF16 = 0, NSF_SEED4 = 1, NSF_Q8 = 2, NSF_Q4 = 3, NSF_SEED4P4 = 4, NSF_SEED6P8 = 5, NSF_TCQ = 8 };
#define NSF_PAGE 16384

typedef struct {
    const uint8_t* p; /* data in the mapping */
    uint64_t len;
    uint64_t off;     /* file offset */
    int shard;
} NsfStream;

/* Streams (nslm/model_st.h:43-44): BF16 0 values; Q8 / Q4 0 packed words, 1 scales, 2 biases; SEED4 0 seeds, 1 nibble
 * words, 2 exponent biases; SEED4P4 / SEED6P8 0 seeds, 1 coefficient words, 2 exponent biases, 3 exponent codes; TCQ 0
 * words, 1 scales (group = L | K << 8 | T << 16). */
typedef struct {
    char name[96];
    int enc, slices, rows, cols;
    int group; /* Q8 / Q4: 64 or 32; TCQ: the packed parameters; else 0 */
    NsfStream s[4];
} NsfTensor;

typedef struct NsfModel NsfModel;

uint64_t nsf_stream_len(int enc, int slices, int rows, int cols, int s); /* ns_stream_len: group 64; 0 = unused stream */
NsfModel* nsf_open(const char* dir, char* err, int errlen);              /* ns_open: the index's shards, else model*.safetensors */
void nsf_close(NsfModel* m);
int nsf_count(const NsfModel* m);
int nsf_shards(const NsfModel* m);
const NsfTensor* nsf_at(const NsfModel* m, int i);                       /* in name order */
const NsfTensor* nsf_find(const NsfModel* m, const char* name);          /* ns_find */
int nsf_mappable(const NsfModel* m, const NsfStream* s);                 /* ns_mappable: page-aligned offset, padded length inside the shard */

/* nslm_blk_stream (nslm/lib_moe.c:92-107): stream s of a whole .blk (p = 3) or .blk4 (p = 4) bank image of E experts
 * [rows][cols] into dst, in the model folder's stream order (codes two a byte, low nibble first).  0, or -1. */
int nsf_blk_stream(const uint8_t* blk, size_t len, int p, int E, int rows, int cols, int s, uint8_t* dst);

/* ---- into HBM (no counterpart in the reference, whose engines map or copy streams one by one) ---- */
/* len bytes of a stream from byte `skip` on, to device memory: staged through two pinned buffers so that reading the
 * mapping overlaps the copies.  0, or -1. */
int nsf_upload(void* dst_dev, const NsfStream* s, uint64_t skip, uint64_t len);

struct NslmMoe;
/* Tensor t (SEED4P4 or SEED4, slices = the layer's experts, [ff][d] for gate / up, [d][ff] for down) as the experts'
 * matrix `which` (0 gate, 1 up, 2 down) of `layer`; the router weight (BF16 [experts][d]) and its optional bias. */
int nslm_moe_load_experts(struct NslmMoe* m, int layer, int which, const NsfTensor* t);
int nslm_moe_load_router(struct NslmMoe* m, int layer, const NsfTensor* w, const NsfTensor* bias);

#ifdef __cplusplus
}
#endif
#endif
