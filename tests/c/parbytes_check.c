/* parbytes_check.c - bt_bytes_equal / bt_bytes_copy against memcmp / memcpy: sizes on both sides of the threshold, a
 * differing byte in every piece and on the piece boundaries, and a forked child (which has no helper threads). */
#include <stdbool.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/wait.h>
#include <unistd.h>

bool bt_bytes_equal(const void* a, const void* b, size_t n);
void bt_bytes_copy(void* dst, const void* src, size_t n);

static uint64_t state = 88172645463325252ull;
static unsigned char next_byte(void) {
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (unsigned char)(state >> 32);
}

static int check(size_t n) {
    unsigned char* a = malloc(n + 64);
    unsigned char* b = malloc(n + 64);
    unsigned char* c = malloc(n + 64);
    if (!a || !b || !c) return 2;
    for (size_t i = 0; i < n + 64; i++) a[i] = next_byte();
    memset(c, 0xA5, n + 64);
    bt_bytes_copy(b + 8, a + 8, n);                       /* unaligned on purpose */
    if (memcmp(a + 8, b + 8, n) != 0) return 3;
    bt_bytes_copy(c + 8, a + 8, n);
    for (size_t i = 0; i < 8; i++) if (c[i] != 0xA5 || c[n + 8 + i] != 0xA5) return 4;   /* nothing outside the range */
    if (!bt_bytes_equal(a + 8, b + 8, n)) return 5;
    if (n == 0) { free(a); free(b); free(c); return 0; }
    const size_t each = (n / 4) & ~(size_t)4095;
    const size_t spots[] = {0, 1, each ? each - 1 : 0, each, 2 * each, each ? 3 * each - 1 : 0, 3 * each, n / 2, n - 2 < n ? n - 2 : 0, n - 1};
    for (size_t s = 0; s < sizeof(spots) / sizeof(spots[0]); s++) {
        const size_t at = spots[s] < n ? spots[s] : n - 1;
        b[8 + at] ^= 0x40;
        if (bt_bytes_equal(a + 8, b + 8, n)) return 6;
        b[8 + at] ^= 0x40;
    }
    if (!bt_bytes_equal(a + 8, b + 8, n)) return 7;
    free(a); free(b); free(c);
    return 0;
}

int main(void) {
    const size_t sizes[] = {0, 1, 4095, 4096, (size_t)1 << 20, ((size_t)2 << 20) - 1, (size_t)2 << 20, ((size_t)2 << 20) + 4097, ((size_t)8 << 20) + 1,
                            ((size_t)33 << 20) + 12345};
    for (size_t i = 0; i < sizeof(sizes) / sizeof(sizes[0]); i++) {
        const int rc = check(sizes[i]);
        if (rc) { printf("size %zu: failure %d\n", sizes[i], rc); return 1; }
    }
    /* many calls in a row (the helpers are reused) */
    for (int rep = 0; rep < 40; rep++)
        if (check(((size_t)2 << 20) + 40960 * (size_t)rep + (size_t)rep)) { printf("repeat %d failed\n", rep); return 1; }
    /* a child of a process whose helpers exist has none: it must still get the right answers */
    const pid_t pid = fork();
    if (pid == 0) _exit(check((size_t)16 << 20) || check((size_t)9 << 20) ? 9 : 0);
    int status = 0;
    if (pid < 0 || waitpid(pid, &status, 0) != pid || !WIFEXITED(status) || WEXITSTATUS(status) != 0) { printf("forked child failed\n"); return 1; }
    printf("ok\n");
    return 0;
}
