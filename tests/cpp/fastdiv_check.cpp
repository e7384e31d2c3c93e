// Host-side check of helix_fastdiv.h: the multiply-shift quotient equals n / d for every divisor the conv
// gathers can meet and dividends up to 2^31 - 1 (strided sweep plus the edges around multiples of d).
#include <stdio.h>

#include "helix_fastdiv.h"

int main() {
    long bad = 0;
    for (int d = 1; d < 3000; d++) {
        const helix_fastdiv::FastDiv f = helix_fastdiv::make(d);
        for (long n = 0; n < 2147483647L; n += 2000003) bad += f.div((int)n) != n / d;
        const int top = 2147483647 / d * d;
        const int edge[] = {0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 2147483647, 2147483646, top, top - 1};
        for (int e : edge)
            if (e >= 0) bad += f.div(e) != e / d;
    }
    const int ds[] = {1, 2, 3, 7, 56, 112, 224, 1 << 20, 1 << 30, 2147483647, 1000003, 65536, 65537};
    for (int d : ds) {
        const helix_fastdiv::FastDiv f = helix_fastdiv::make(d);
        for (long n = 0; n < 2147483647L; n += 99991) bad += f.div((int)n) != n / d;
        bad += f.div(2147483647) != 2147483647 / d;
    }
    printf("mismatches %ld\n", bad);
    return bad != 0;
}
