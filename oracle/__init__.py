"""CPU oracle for the block-quantized weight path. Test infrastructure only."""
