/* Tensor-layout functions (library and header-inline) against the cases of the reference's own unit test
 * (tests/nvcv_types/system/TestTensorLayout.cpp:30-480), restated. Built and run by tests/test_core.py against
 * libnvcv_types.so; prints one line per failed case and returns their number. */
#include <nvcv/TensorLayout.h>

#include <stdio.h>
#include <string.h>

static int failures = 0;
#define CHECK(cond)                                               \
    do                                                            \
    {                                                             \
        if (!(cond))                                              \
        {                                                         \
            printf("line %d: %s\n", __LINE__, #cond);             \
            ++failures;                                           \
        }                                                         \
    }                                                             \
    while (0)

static NVCVTensorLayout L(const char *s)
{
    NVCVTensorLayout l;
    if (nvcvTensorLayoutMake(s, &l) != NVCV_SUCCESS)
    {
        printf("cannot make layout %s\n", s);
        ++failures;
        memset(&l, 0, sizeof(l));
    }
    return l;
}

static int Same(NVCVTensorLayout a, const char *gold)
{
    return a.rank == (int)strlen(gold) && memcmp(a.data, gold, strlen(gold)) == 0;
}

int main(void)
{
    NVCVTensorLayout t;
    /* make, from string and from range (:30-66) */
    const char *strs[] = {"ABC", "", "0123456789ABCDE"};
    for (int i = 0; i < 3; ++i)
    {
        CHECK(nvcvTensorLayoutMake(strs[i], &t) == NVCV_SUCCESS && Same(t, strs[i]));
        CHECK(nvcvTensorLayoutMakeRange(strs[i], strs[i] + strlen(strs[i]), &t) == NVCV_SUCCESS && Same(t, strs[i]));
        const NVCVTensorLayout macro = NVCV_TENSOR_LAYOUT_MAKE("0123456789ABCDE");
        CHECK(i != 2 || (nvcvTensorLayoutCompare(macro, t) == 0 && macro.rank == 15));
    }
    CHECK(nvcvTensorLayoutMake(NULL, &t) == NVCV_SUCCESS && t.rank == 0);

    /* first / last n labels, negative n counts from the other end (:69-130) */
    const struct { int n; const char *first, *last; } fl[] = {
        {0, "", ""}, {1, "A", "C"}, {2, "AB", "BC"}, {3, "ABC", "ABC"}, {4, "ABC", "ABC"},
        {-1, "C", "A"}, {-2, "BC", "AB"}, {-3, "ABC", "ABC"}, {-4, "ABC", "ABC"}};
    for (unsigned i = 0; i < sizeof(fl) / sizeof(fl[0]); ++i)
    {
        CHECK(nvcvTensorLayoutMakeFirst(L("ABC"), fl[i].n, &t) == NVCV_SUCCESS && Same(t, fl[i].first));
        CHECK(nvcvTensorLayoutMakeLast(L("ABC"), fl[i].n, &t) == NVCV_SUCCESS && Same(t, fl[i].last));
    }

    /* sub-ranges (:133-185) */
    const struct { int beg, end; const char *gold; } sr[] = {
        {0, 0, ""}, {0, 1, "A"}, {0, 3, "ABC"}, {0, 4, "ABCD"}, {0, 5, "ABCD"}, {-1, 0, ""}, {1, 1, ""}, {1, 2, "B"},
        {1, 3, "BC"}, {3, 4, "D"}, {3, 5, "D"}, {4, 5, ""}, {5, 7, ""}, {-2, -1, "C"}, {-3, -1, "BC"}, {-3, -3, ""},
        {-1, -2, ""}, {-4, -3, "A"}, {-5, -3, "A"}, {-5, -5, ""}, {-6, -5, ""}, {-4, -1, "ABC"}, {-4, 4, "ABCD"},
        {-3, 4, "BCD"}, {1, -1, "BC"}};
    for (unsigned i = 0; i < sizeof(sr) / sizeof(sr[0]); ++i)
    {
        CHECK(nvcvTensorLayoutMakeSubRange(L("ABCD"), sr[i].beg, sr[i].end, &t) == NVCV_SUCCESS && Same(t, sr[i].gold));
        if (!Same(t, sr[i].gold))
        {
            printf("  sub-range %d..%d gave rank %d\n", sr[i].beg, sr[i].end, t.rank);
        }
    }

    /* find (:187-216) */
    const struct { char label; int start, gold; } fd[] = {{'C', 0, 2}, {'C', 2, 2}, {'C', 3, -1}, {'z', 0, -1}, {'D', 0, 3},
                                                         {'A', 0, 0}, {'D', -2, 3}, {'D', -1, 3}, {'C', -1, -1}};
    for (unsigned i = 0; i < sizeof(fd) / sizeof(fd[0]); ++i)
    {
        CHECK(nvcvTensorLayoutFindDimIndex(L("ABCD"), fd[i].label, fd[i].start) == fd[i].gold);
    }

    /* label at an index (:219-247) */
    const struct { int idx; char gold; } gl[] = {{0, 'A'}, {1, 'B'}, {3, 'D'}, {4, 0}, {5, 0}, {-1, 'D'}, {-2, 'C'}, {-4, 'A'}, {-5, 0}, {-6, 0}};
    for (unsigned i = 0; i < sizeof(gl) / sizeof(gl[0]); ++i)
    {
        CHECK(nvcvTensorLayoutGetLabel(L("ABCD"), gl[i].idx) == gl[i].gold);
    }

    /* rank (:250-272) */
    CHECK(nvcvTensorLayoutGetNumDim(L("ABCD")) == 4 && nvcvTensorLayoutGetNumDim(L("")) == 0 && nvcvTensorLayoutGetNumDim(L(".")) == 1);
    {
        const NVCVTensorLayout nul = NVCV_TENSOR_LAYOUT_MAKE("\0"); /* one dimension labelled NUL */
        CHECK(nvcvTensorLayoutGetNumDim(nul) == 1);
        CHECK(nvcvTensorLayoutCompare(L("A"), nul) == 'A' && nvcvTensorLayoutCompare(nul, L("A")) == -'A');
        CHECK(strcmp(nvcvTensorLayoutGetName(&nul), "") == 0);
    }
    CHECK(nvcvTensorLayoutGetNumDim(L("0123456789ABCDE")) == 15);

    /* compare (:274-302) */
    CHECK(nvcvTensorLayoutCompare(L("ABCD"), L("ABCD")) == 0 && nvcvTensorLayoutCompare(L(""), L("")) == 0);
    CHECK(nvcvTensorLayoutCompare(L("ABC"), L("ABD")) == -1 && nvcvTensorLayoutCompare(L("ABC"), L("ABB")) == 1);
    CHECK(nvcvTensorLayoutCompare(L("A"), L("ABC")) == -2 && nvcvTensorLayoutCompare(L("ABC"), L("A")) == 2);
    CHECK(nvcvTensorLayoutCompare(L(""), L("ABC")) == -3 && nvcvTensorLayoutCompare(L("ABC"), L("")) == 3);

    /* name (:305-330) */
    const char *names[] = {"ABCD", "", "0", "0123456789ABCDE", " AB", "AB ", "A B"};
    for (int i = 0; i < 7; ++i)
    {
        const NVCVTensorLayout l = L(names[i]);
        CHECK(strcmp(nvcvTensorLayoutGetName(&l), names[i]) == 0);
    }

    /* starts with / ends with (:333-397) */
    const struct { const char *a, *b; int starts; } sw[] = {{"A", "A", 1}, {"ABCD", "ABCD", 1}, {"ABCD", "ABC", 1}, {"ABCD", "A", 1},
        {"", "", 1}, {"23l2", "", 1}, {"ABCD", "ACD", 0}, {"ABCD", "ABCDE", 0}, {"A", "E", 0}, {"AE", "E", 0}, {"AE", "EA", 0}};
    for (unsigned i = 0; i < sizeof(sw) / sizeof(sw[0]); ++i)
    {
        CHECK((nvcvTensorLayoutStartsWith(L(sw[i].a), L(sw[i].b)) != 0) == sw[i].starts);
    }
    const struct { const char *a, *b; int ends; } ew[] = {{"A", "A", 1}, {"ABCD", "ABCD", 1}, {"ABCD", "BCD", 1}, {"ABCD", "D", 1},
        {"", "", 1}, {"23l2", "", 1}, {"ABCD", "ACD", 0}, {"ABCD", "ZABCD", 0}, {"A", "E", 0}, {"AE", "A", 0}, {"AE", "EA", 0}};
    for (unsigned i = 0; i < sizeof(ew) / sizeof(ew[0]); ++i)
    {
        CHECK((nvcvTensorLayoutEndsWith(L(ew[i].a), L(ew[i].b)) != 0) == ew[i].ends);
    }

    /* invalid arguments (:428-475) */
    char exceeded[NVCV_TENSOR_MAX_RANK + 2], valid[NVCV_TENSOR_MAX_RANK];
    memset(exceeded, 'Z', NVCV_TENSOR_MAX_RANK + 1);
    exceeded[NVCV_TENSOR_MAX_RANK + 1] = 0;
    memset(valid, 'Z', NVCV_TENSOR_MAX_RANK - 1);
    valid[NVCV_TENSOR_MAX_RANK - 1] = 0;
    CHECK(nvcvTensorLayoutMake("HW", NULL) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMake(exceeded, &t) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeRange(valid, valid + strlen(valid), NULL) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeRange(NULL, valid + strlen(valid), &t) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeRange(valid, NULL, &t) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeRange(exceeded, exceeded + strlen(exceeded), &t) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeRange(valid + 1, valid, &t) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeFirst(L("ABCD"), 2, NULL) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeLast(L("ABCD"), 2, NULL) == NVCV_ERROR_INVALID_ARGUMENT);
    CHECK(nvcvTensorLayoutMakeSubRange(L("ABCD"), 0, 2, NULL) == NVCV_ERROR_INVALID_ARGUMENT);
    printf("%d failures\n", failures);
    return failures;
}
