"""CPU oracle for the quantized linear-layer path.  Test infrastructure only: nothing in the shipped
package imports this module."""
