"""Which bytes the bilinear kernels' tap accesses touch, worked out on the CPU for small, tight-pitch, odd-aligned images.

The kernels fetch the two horizontally adjacent taps of a pixel as ONE dword-aligned window: it starts at the dword
boundary at or below the first tap and is 12 bytes long for 3-byte pixels (include/fkd/ops.hpp, PairWindow), so it can
reach up to 6 bytes past the second tap.  Two rules keep that inside the allocation, and torch's padded allocations
would hide a violation on the GPU, so they are checked here by brute force over every tap position:

* tile form (k_gather): waves whose taps reach a row with (height - 1 - y) * pitch < 8 bytes of image behind its start
  take one access per channel instead (Read2D::tap_row / tap_last); every other window must end inside the image;
* strip form (k_strip): the buffer resource ends with the dword that holds the image's last byte (make_tap_image with a
  size); dwords at or beyond that extent are not fetched (they read as zero).  Every byte a blend USES must lie in a
  delivered dword, and every delivered dword must start inside the image, so that it lies in a mapped page.
"""
import itertools

ELEM = 3          # bytes per pixel (uchar3)
WINDOW = 12       # dwords fetched per pair window: 3


def _image_bytes(w, h, pitch):
    return pitch * (h - 1) + w * ELEM


def _cases():
    for w, h in itertools.product((2, 3, 5, 8, 11), (1, 2, 3, 5)):
        for pad in (0, 1, 2, 3, 5):
            for lo in (0, 1, 2, 3):               # offset of the image's first byte inside its dword
                yield w, h, w * ELEM + pad, lo


def test_tile_form_windows_stay_inside_the_image():
    checked = 0
    for w, h, pitch, lo in _cases():
        size = _image_bytes(w, h, pitch)
        for y in range(h):
            last = (h - 1 - y) * pitch < 8                      # Read2D::tap_row
            for x1 in range(w - 1):                             # first tap; the second one is x1 + 1 <= w - 1
                first_byte = y * pitch + x1 * ELEM              # relative to the image's first byte
                if last:
                    touched = range(first_byte, first_byte + 2 * ELEM)          # channel by channel, nothing else
                else:
                    start = ((lo + first_byte) & ~3) - lo       # the dword at or below the first tap (rows of any alignment)
                    touched = range(start, start + WINDOW)
                    # a window may begin up to 3 bytes before its first tap: the same dword as a byte that is needed
                    assert first_byte - start <= 3
                assert touched[-1] < size, (w, h, pitch, lo, y, x1)
                assert touched[0] >= -3                         # at most the image's own first dword
                checked += 1
    assert checked > 5000


def test_strip_form_extent_delivers_every_used_byte_and_nothing_unmapped():
    for w, h, pitch, lo in _cases():
        if pitch % 4:
            continue                                            # the strip form is only launched for pitches that are multiples of 4
        size = _image_bytes(w, h, pitch)
        extent = (size + lo + 3) & ~3                           # make_tap_image(data, bytes): relative to the dword-aligned base
        # every delivered dword starts inside the image (so it shares a page with image bytes)
        assert extent - 4 < lo + size
        for y in range(h):
            for x1 in range(w - 1):
                first_byte = lo + y * pitch + x1 * ELEM         # relative to the resource's base
                start = first_byte & ~3
                used = range(first_byte, first_byte + 2 * ELEM)
                for b in used:
                    assert (b & ~3) + 4 <= extent, (w, h, pitch, lo, y, x1)     # its dword is inside the extent: delivered
                assert start + WINDOW <= extent + 8             # at most two dwords of a window are beyond the extent (read as zero)
