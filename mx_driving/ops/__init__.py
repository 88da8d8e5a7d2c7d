"""``mx_driving.ops`` -- module paths of the reference's operator layer for the operators this repository provides
(mx_driving/__init__.py:84-151 of the reference imports from ``.ops.<operator>``)."""
