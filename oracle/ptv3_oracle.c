/* Scalar C restatement of the integer half of the PTv3 forward path.
 *
 * TEST INFRASTRUCTURE: this file is the checker and the timed CPU baseline. Nothing in
 * the shipped package links or loads it.
 *
 * Each function cites the reference lines it restates (paths relative to the reference
 * checkout). The code is written per point on machine words; the reference works on
 * whole tensors of single bits.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- z-order: serialization/z_order.py:40-50 (bit i of x,y,z -> bits 3i+2,3i+1,3i),
 *      coordinates masked to `depth` bits as in z_order.py:90-94. */
static uint64_t z_code(uint64_t x, uint64_t y, uint64_t z, int depth) {
    uint64_t key = 0;
    for (int i = 0; i < depth; ++i) {
        key |= ((x >> i) & 1ull) << (3 * i + 2);
        key |= ((y >> i) & 1ull) << (3 * i + 1);
        key |= ((z >> i) & 1ull) << (3 * i);
    }
    return key;
}

/* ---- Hilbert: serialization/hilbert.py:154-181. Skilling's AxestoTranspose walks the
 *      levels from the most significant one down; the Gray decode of :69-88 is a prefix
 *      XOR over the interleaved word, done here one bit at a time from the top. */
static uint64_t hilbert_code(uint64_t x, uint64_t y, uint64_t z, int depth) {
    uint64_t X[3] = {x, y, z};
    for (int q = depth - 1; q >= 0; --q) {
        const uint64_t Q = 1ull << q, P = Q - 1;
        for (int i = 0; i < 3; ++i) {
            if (X[i] & Q) {
                X[0] ^= P; /* hilbert.py:160-165 */
            } else {
                const uint64_t t = (X[0] ^ X[i]) & P; /* hilbert.py:168-175 */
                X[0] ^= t;
                X[i] ^= t;
            }
        }
    }
    uint64_t h = 0;
    unsigned acc = 0; /* running parity = binary bit (prefix XOR of Gray bits) */
    for (int b = depth - 1; b >= 0; --b) {
        for (int i = 0; i < 3; ++i) { /* axis 0 is the most significant of a level, :178 */
            acc ^= (unsigned)((X[i] >> b) & 1ull);
            h = (h << 1) | acc;
        }
    }
    return h;
}

/* ---- serialization/default.py:8-24. order_id: 0 z, 1 z-trans, 2 hilbert, 3 hilbert-trans.
 *      grid_coord is (n,3) int32 row-major, batch may be NULL. */
int orc_encode(const int32_t *grid_coord, const int64_t *batch, int64_t n, int depth,
               int order_id, int64_t *code) {
    if (depth < 1 || depth > 21 || order_id < 0 || order_id > 3) return -1;
    const uint64_t mask = (1ull << depth) - 1;
    for (int64_t p = 0; p < n; ++p) {
        uint64_t x = (uint64_t)(int64_t)grid_coord[3 * p + 0] & mask;
        uint64_t y = (uint64_t)(int64_t)grid_coord[3 * p + 1] & mask;
        uint64_t z = (uint64_t)(int64_t)grid_coord[3 * p + 2] & mask;
        if (order_id & 1) { uint64_t t = x; x = y; y = t; } /* default.py:14,18 */
        uint64_t c = (order_id < 2) ? z_code(x, y, z, depth) : hilbert_code(x, y, z, depth);
        if (batch) c |= (uint64_t)batch[p] << (3 * depth); /* default.py:21-23 */
        code[p] = (int64_t)c;
    }
    return 0;
}

/* ---- Submanifold kernel map, the canonical form of what spconv builds for
 *      SubMConv3d (call sites model.py:546-552, :767-774): for voxel i and kernel
 *      offset k = (kx*ks + ky)*ks + kz, nbr[i*V + k] = index of the voxel at
 *      (b, x+kx-r, y+ky-r, z+kz-r) or -1, r = ks/2, V = ks^3.
 *      indices is (n,4) int32 [b,x,y,z] as in model.py:167-169. Sort + binary search. */
typedef struct { uint64_t key; int32_t idx; } kv_t;
static int kv_cmp(const void *a, const void *b) {
    const uint64_t x = ((const kv_t *)a)->key, y = ((const kv_t *)b)->key;
    return (x > y) - (x < y);
}
static uint64_t vox_key(int64_t b, int64_t x, int64_t y, int64_t z) {
    /* 17 bits per axis after a +4 shift keeps neighbours of coordinate 0 distinct */
    return ((uint64_t)b << 51) | ((uint64_t)(x + 4) << 34) | ((uint64_t)(y + 4) << 17) |
           (uint64_t)(z + 4);
}
int orc_kmap(const int32_t *indices, int64_t n, int ks, int32_t *nbr) {
    if (ks != 3 && ks != 5) return -1;
    kv_t *tab = (kv_t *)malloc(sizeof(kv_t) * (size_t)(n > 0 ? n : 1));
    if (!tab) return -2;
    for (int64_t i = 0; i < n; ++i) {
        const int32_t *v = indices + 4 * i;
        tab[i].key = vox_key(v[0], v[1], v[2], v[3]);
        tab[i].idx = (int32_t)i;
    }
    qsort(tab, (size_t)n, sizeof(kv_t), kv_cmp);
    const int r = ks / 2, V = ks * ks * ks;
    for (int64_t i = 0; i < n; ++i) {
        const int32_t *v = indices + 4 * i;
        for (int kx = 0; kx < ks; ++kx)
            for (int ky = 0; ky < ks; ++ky)
                for (int kz = 0; kz < ks; ++kz) {
                    const uint64_t key =
                        vox_key(v[0], (int64_t)v[1] + kx - r, (int64_t)v[2] + ky - r,
                                (int64_t)v[3] + kz - r);
                    int64_t lo = 0, hi = n;
                    while (lo < hi) {
                        const int64_t mid = (lo + hi) >> 1;
                        if (tab[mid].key < key) lo = mid + 1; else hi = mid;
                    }
                    nbr[i * V + (kx * ks + ky) * ks + kz] =
                        (lo < n && tab[lo].key == key) ? tab[lo].idx : -1;
                }
    }
    free(tab);
    return 0;
}
